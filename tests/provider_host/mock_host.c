/* Test double of the runtime side of the provider SPI
 * (native/include/volvoxai_backend.h): accepts a registration under the same
 * descriptor checks as the reference (native/src/runtime/backend_sdk.c:96-139),
 * then drives one package through runtime_create -> compile -> context_create
 * -> context_execute -> destroy the way the reference's lifecycle does, holding
 * the provider to the contract: identities echoed, route attested, every
 * declared output written exactly once with the exact name, dtype and shape.
 * Test infrastructure only. */
#include "volvoxai_backend.h"

#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

static VxBackendProvider g_provider;
static char g_name[VX_BACKEND_NAME_CAPACITY];
static int g_registered;

static int name_valid(const char* name) {
    size_t length;
    if (!name || !name[0]) return 0;
    length = strlen(name);
    if (length >= VX_BACKEND_NAME_CAPACITY || name[0] < 'a' || name[0] > 'z') return 0;
    for (size_t i = 1; i < length; i++) {
        unsigned char c = (unsigned char)name[i];
        if (!((c >= 'a' && c <= 'z') || (c >= '0' && c <= '9') || c == '.' || c == '_' || c == '-')) return 0;
    }
    return strcmp(name, "cpu") && strcmp(name, "cuda") && strcmp(name, "vulkan") && strcmp(name, "metal");
}

VX_API VxStatus vx_backend_register_provider(const VxBackendProvider* p, VxReport* report) {
    if (!report || report->struct_size != sizeof(*report)) return VX_STATUS_INVALID_ARGUMENT;
    if (p && p->struct_size == sizeof(*p) && p->abi_version != VX_BACKEND_ABI_VERSION) return VX_STATUS_ABI_UNSUPPORTED;
    if (!p || p->struct_size != sizeof(*p) || p->exact_contract_marker != VX_BACKEND_PROVIDER_EXACT_CONTRACT_MARKER ||
        p->exact_contract_extent != sizeof(*p) || !name_valid(p->name) || p->flags != 0 ||
        p->shape_domain.struct_size != sizeof(p->shape_domain) || !p->shape_domain.proof_protocol ||
        !p->shape_domain.resource_protocol ||
        strcmp(p->shape_domain.proof_protocol, VX_BACKEND_SHAPE_PROOF_PROTOCOL) ||
        strcmp(p->shape_domain.resource_protocol, VX_BACKEND_RESOURCE_PROTOCOL) ||
        (p->shape_domain.support != VX_BACKEND_SHAPE_DOMAIN_FULL &&
         p->shape_domain.support != VX_BACKEND_SHAPE_DOMAIN_UNSUPPORTED) ||
        !p->runtime_create || !p->runtime_destroy || !p->compile || !p->compiled_destroy ||
        (!!p->compiled_batch_contract != !!p->context_execute_batch) || !p->context_create || !p->context_execute ||
        !p->context_destroy)
        return VX_STATUS_INVALID_ARGUMENT;
    if (g_registered && !strcmp(g_name, p->name)) return VX_STATUS_INVALID_ARGUMENT; /* duplicate */
    g_provider = *p;
    snprintf(g_name, sizeof(g_name), "%s", p->name);
    g_provider.name = g_name;
    g_registered = 1;
    report->status = VX_STATUS_OK;
    return VX_STATUS_OK;
}

/* Calls a provider's registration function with a report of the right layout. */
int32_t mock_host_register(VxStatus (*register_provider)(VxReport*)) {
    VxReport report = VX_REPORT_INIT;
    return register_provider ? (int32_t)register_provider(&report) : (int32_t)VX_STATUS_INVALID_ARGUMENT;
}

const char* mock_host_registered_name(void) { return g_registered ? g_name : ""; }
uint32_t mock_host_shape_domain_support(void) { return g_registered ? g_provider.shape_domain.support : 0u; }

typedef struct MockRun {
    /* in */
    const char* graph_path;
    const char* weight_path;
    int32_t packed_arithmetic;
    const char* input_name;
    int32_t input_dtype;
    uint32_t rank;
    int64_t input_shape[VX_MAX_TENSOR_RANK];
    int64_t lead_max[VX_MAX_TENSOR_RANK]; /* > 0: that leading axis is symbolic, bounded 1..lead_max */
    const void* input;
    uint64_t input_bytes;
    const char* output_name;
    int32_t output_dtype;
    int64_t output_last;
    void* output;
    uint64_t output_capacity;
    int32_t executions;
    /* out */
    int32_t status;
    int32_t failed_stage; /* VxStage of the callback that failed */
    uint64_t output_bytes;
    int32_t writes;
    int32_t sink_mismatch;
    int32_t compile_attested, execute_attested, identities_echoed, attested_arithmetic;
    uint64_t maximum_tensor_bytes, maximum_resident_bytes;
    char message[VX_REPORT_MESSAGE_CAPACITY];
    char compile_route[VX_REPORT_ROUTE_CAPACITY];
    char execute_route[VX_REPORT_ROUTE_CAPACITY];
    char device[VX_REPORT_DEVICE_CAPACITY];
} MockRun;

static VxStatus sink_write(void* user, const char* name, VxDataType dtype, const int64_t* shape, uint32_t rank,
                           const void* data, size_t bytes) {
    MockRun* run = (MockRun*)user;
    run->writes++;
    if (!name || strcmp(name, run->output_name) || (int32_t)dtype != run->output_dtype || rank != run->rank || !data ||
        bytes > run->output_capacity || shape[rank - 1] != run->output_last) {
        run->sink_mismatch = 1;
        return VX_STATUS_INVALID_ARGUMENT;
    }
    for (uint32_t a = 0; a + 1 < rank; a++)
        if (shape[a] != run->input_shape[a]) {
            run->sink_mismatch = 1;
            return VX_STATUS_INVALID_ARGUMENT;
        }
    memcpy(run->output, data, bytes); /* the sink copies before write returns */
    run->output_bytes = bytes;
    return VX_STATUS_OK;
}

static void spec_from(VxTensorSpec* spec, const char* name, int32_t dtype, const MockRun* run, int64_t last) {
    memset(spec, 0, sizeof(*spec));
    spec->struct_size = sizeof(*spec);
    spec->name = name;
    spec->dtype = (VxDataType)dtype;
    spec->rank = run->rank;
    spec->location = VX_MEMORY_HOST;
    for (uint32_t a = 0; a < run->rank; a++) {
        VxDimensionConstraint* d = &spec->dimensions[a];
        d->struct_size = sizeof(*d);
        d->multiple_of = 1;
        if (a + 1 < run->rank && run->lead_max[a] > 0) {
            d->kind = VX_DIMENSION_SYMBOLIC;
            d->symbol = "rows";
            d->min = 1;
            d->max = run->lead_max[a];
        } else {
            d->kind = VX_DIMENSION_FIXED;
            d->symbol = NULL;
            d->min = d->max = a + 1 < run->rank ? run->input_shape[a] : last;
        }
    }
}

int32_t mock_host_run(MockRun* run) {
    static const char fingerprint[] = "sha256:mock-graph-fingerprint";
    static const char proof[] = "sha256:mock-shape-domain-proof";
    VxRuntimeOptions runtime_options = VX_RUNTIME_OPTIONS_INIT;
    VxContextOptions context_options = VX_CONTEXT_OPTIONS_INIT;
    VxReport report = VX_REPORT_INIT;
    VxModelSource source = VX_MODEL_SOURCE_INIT;
    VxBackendCompileInput input = VX_BACKEND_COMPILE_INPUT_INIT;
    VxBackendShapeDomainAttestation attestation = VX_BACKEND_SHAPE_DOMAIN_ATTESTATION_INIT;
    VxBackendPolicy policy = VX_BACKEND_POLICY_INIT;
    VxTensorSpec in_spec, out_spec;
    VxTensorBinding binding = VX_TENSOR_BINDING_INIT;
    VxBackendOutputSink sink = {sizeof(VxBackendOutputSink), run, sink_write};
    const char* weights[1];
    const char* wanted[1];
    void *runtime = NULL, *compiled = NULL, *context = NULL;
    VxStatus status;
    if (!g_registered) return run->status = VX_STATUS_NOT_FOUND;
    run->writes = 0;
    run->sink_mismatch = 0;

    status = g_provider.runtime_create(g_provider.user_data, &runtime_options, &runtime, &report);
    run->failed_stage = VX_STAGE_RUNTIME_CREATE;
    if (status != VX_STATUS_OK) goto done;

    weights[0] = run->weight_path;
    source.graph_path = run->graph_path;
    source.weight_paths = weights;
    source.weight_path_count = 1;
    spec_from(&in_spec, run->input_name, run->input_dtype, run, run->input_shape[run->rank - 1]);
    spec_from(&out_spec, run->output_name, run->output_dtype, run, run->output_last);
    input.source = &source;
    input.graph_fingerprint = fingerprint;
    input.shape_domain_proof_identity = proof;
    input.inputs = &in_spec;
    input.input_count = 1;
    input.outputs = &out_spec;
    input.output_count = 1;
    input.packed_arithmetic = (VxPackedArithmetic)run->packed_arithmetic;
    wanted[0] = g_name;
    policy.mode = VX_BACKEND_REQUIRE;
    policy.operator_fallback = VX_OPERATOR_FALLBACK_FORBID;
    policy.backends = wanted;
    policy.backend_count = 1;
    report = (VxReport)VX_REPORT_INIT;
    status = g_provider.compile(runtime, &input, &policy, &compiled, &attestation, &report);
    run->failed_stage = VX_STAGE_COMPILE;
    if (status != VX_STATUS_OK) {
        if (compiled) status = VX_STATUS_INTERNAL; /* a failed compile must not leave an instance */
        goto done;
    }
    run->compile_attested = report.route_attested && !report.operator_fallback_used && report.route_evidence[0] &&
                            report.device[0];
    snprintf(run->compile_route, sizeof(run->compile_route), "%s", report.route_evidence);
    snprintf(run->device, sizeof(run->device), "%s", report.device);
    run->identities_echoed = attestation.graph_fingerprint && attestation.shape_domain_proof_identity &&
                             !strcmp(attestation.graph_fingerprint, fingerprint) &&
                             !strcmp(attestation.shape_domain_proof_identity, proof);
    run->attested_arithmetic = attestation.packed_arithmetic;
    run->maximum_tensor_bytes = attestation.maximum_tensor_bytes;
    run->maximum_resident_bytes = attestation.maximum_resident_bytes;

    report = (VxReport)VX_REPORT_INIT;
    status = g_provider.context_create(compiled, &context_options, &context, &report);
    run->failed_stage = VX_STAGE_CONTEXT_CREATE;
    if (status != VX_STATUS_OK) goto done;

    binding.name = run->input_name;
    binding.dtype = (VxDataType)run->input_dtype;
    binding.rank = run->rank;
    memcpy(binding.shape, run->input_shape, sizeof(binding.shape));
    binding.data = run->input;
    binding.byte_size = (size_t)run->input_bytes;
    binding.location = VX_MEMORY_HOST;
    run->failed_stage = VX_STAGE_EXECUTE;
    for (int32_t i = 0; i < (run->executions > 0 ? run->executions : 1) && status == VX_STATUS_OK; i++) {
        const int32_t before = run->writes;
        report = (VxReport)VX_REPORT_INIT;
        status = g_provider.context_execute(context, &binding, 1, &sink, &report);
        if (status == VX_STATUS_OK && (run->writes != before + 1 || run->sink_mismatch)) status = VX_STATUS_EXECUTION_FAILED;
        run->execute_attested = report.route_attested && report.route_evidence[0];
        snprintf(run->execute_route, sizeof(run->execute_route), "%s", report.route_evidence);
    }
    if (status == VX_STATUS_OK) run->failed_stage = VX_STAGE_NONE;

done:
    snprintf(run->message, sizeof(run->message), "%s", report.message);
    if (context) {
        if (g_provider.context_close) (void)g_provider.context_close(context, &report);
        g_provider.context_destroy(context);
    }
    if (compiled) g_provider.compiled_destroy(compiled);
    if (runtime) g_provider.runtime_destroy(runtime);
    return run->status = status;
}

/* Several contexts of ONE compiled instance executing at the same time on their own threads
 * (native/tests/test_packed_arithmetic.inc:128-147): every thread must deliver the bytes a
 * single-threaded run delivers.  run->output receives thread 0's result. */
typedef struct Worker {
    MockRun run; /* private copy: own sink state and output buffer */
    void* compiled;
    VxStatus status;
} Worker;

static void* worker_main(void* opaque) {
    Worker* w = (Worker*)opaque;
    VxContextOptions context_options = VX_CONTEXT_OPTIONS_INIT;
    VxTensorBinding binding = VX_TENSOR_BINDING_INIT;
    VxBackendOutputSink sink = {sizeof(VxBackendOutputSink), &w->run, sink_write};
    VxReport report = VX_REPORT_INIT;
    void* context = NULL;
    w->status = g_provider.context_create(w->compiled, &context_options, &context, &report);
    if (w->status != VX_STATUS_OK) return NULL;
    binding.name = w->run.input_name;
    binding.dtype = (VxDataType)w->run.input_dtype;
    binding.rank = w->run.rank;
    memcpy(binding.shape, w->run.input_shape, sizeof(binding.shape));
    binding.data = w->run.input;
    binding.byte_size = (size_t)w->run.input_bytes;
    binding.location = VX_MEMORY_HOST;
    for (int32_t i = 0; i < w->run.executions && w->status == VX_STATUS_OK; i++) {
        report = (VxReport)VX_REPORT_INIT;
        w->status = g_provider.context_execute(context, &binding, 1, &sink, &report);
        if (w->status == VX_STATUS_OK && (w->run.writes != i + 1 || w->run.sink_mismatch))
            w->status = VX_STATUS_EXECUTION_FAILED;
    }
    g_provider.context_destroy(context);
    return NULL;
}

int32_t mock_host_run_concurrent(MockRun* run, int32_t threads) {
    static const char fingerprint[] = "sha256:mock-graph-fingerprint";
    static const char proof[] = "sha256:mock-shape-domain-proof";
    VxRuntimeOptions runtime_options = VX_RUNTIME_OPTIONS_INIT;
    VxReport report = VX_REPORT_INIT;
    VxModelSource source = VX_MODEL_SOURCE_INIT;
    VxBackendCompileInput input = VX_BACKEND_COMPILE_INPUT_INIT;
    VxBackendShapeDomainAttestation attestation = VX_BACKEND_SHAPE_DOMAIN_ATTESTATION_INIT;
    VxBackendPolicy policy = VX_BACKEND_POLICY_INIT;
    VxTensorSpec in_spec, out_spec;
    const char* weights[1];
    const char* wanted[1];
    void *runtime = NULL, *compiled = NULL;
    Worker* workers;
    pthread_t* ids;
    VxStatus status;
    if (!g_registered || threads < 1 || threads > 16) return run->status = VX_STATUS_INVALID_ARGUMENT;
    status = g_provider.runtime_create(g_provider.user_data, &runtime_options, &runtime, &report);
    if (status != VX_STATUS_OK) return run->status = status;
    weights[0] = run->weight_path;
    source.graph_path = run->graph_path;
    source.weight_paths = weights;
    source.weight_path_count = 1;
    spec_from(&in_spec, run->input_name, run->input_dtype, run, run->input_shape[run->rank - 1]);
    spec_from(&out_spec, run->output_name, run->output_dtype, run, run->output_last);
    input.source = &source;
    input.graph_fingerprint = fingerprint;
    input.shape_domain_proof_identity = proof;
    input.inputs = &in_spec;
    input.input_count = 1;
    input.outputs = &out_spec;
    input.output_count = 1;
    input.packed_arithmetic = (VxPackedArithmetic)run->packed_arithmetic;
    wanted[0] = g_name;
    policy.mode = VX_BACKEND_REQUIRE;
    policy.operator_fallback = VX_OPERATOR_FALLBACK_FORBID;
    policy.backends = wanted;
    policy.backend_count = 1;
    status = g_provider.compile(runtime, &input, &policy, &compiled, &attestation, &report);
    if (status != VX_STATUS_OK) {
        g_provider.runtime_destroy(runtime);
        return run->status = status;
    }
    workers = (Worker*)calloc((size_t)threads, sizeof(*workers));
    ids = (pthread_t*)calloc((size_t)threads, sizeof(*ids));
    for (int32_t t = 0; t < threads; t++) {
        workers[t].run = *run;
        workers[t].run.writes = 0;
        workers[t].run.sink_mismatch = 0;
        workers[t].run.executions = run->executions > 0 ? run->executions : 1;
        workers[t].run.output = malloc((size_t)run->output_capacity);
        workers[t].compiled = compiled;
        pthread_create(&ids[t], NULL, worker_main, &workers[t]);
    }
    for (int32_t t = 0; t < threads; t++) {
        pthread_join(ids[t], NULL);
        if (status == VX_STATUS_OK) status = workers[t].status;
        if (status == VX_STATUS_OK && (workers[t].run.output_bytes != workers[0].run.output_bytes ||
                                       memcmp(workers[t].run.output, workers[0].run.output,
                                              (size_t)workers[0].run.output_bytes) != 0))
            status = VX_STATUS_EXECUTION_FAILED;
    }
    if (status == VX_STATUS_OK) {
        memcpy(run->output, workers[0].run.output, (size_t)workers[0].run.output_bytes);
        run->output_bytes = workers[0].run.output_bytes;
        run->writes = workers[0].run.writes;
    }
    for (int32_t t = 0; t < threads; t++) free(workers[t].run.output);
    free(workers);
    free(ids);
    g_provider.compiled_destroy(compiled);
    g_provider.runtime_destroy(runtime);
    return run->status = status;
}

/* Scheduler-style batch: the provider freezes a batch contract at compile and then receives ONE
 * invocation with the requests stacked along the batch axis, one output sink per lane
 * (native/include/volvoxai_backend.h:39-92; contract checks as in
 * native/src/runtime/public_api_model_lifecycle.inc:790-849).  run->input is the stacked input
 * [batch, ..., d_in] (input_shape[0] == batch, lead_max[0] the symbolic bound); lane i's output
 * lands at run->output + i * lane_bytes. */
typedef struct Lane {
    MockRun* run;
    unsigned char* dst;
    size_t capacity;
    int32_t writes;
    int32_t mismatch;
    size_t bytes;
} Lane;

static VxStatus lane_write(void* user, const char* name, VxDataType dtype, const int64_t* shape, uint32_t rank,
                           const void* data, size_t bytes) {
    Lane* lane = (Lane*)user;
    const MockRun* run = lane->run;
    lane->writes++;
    if (!name || strcmp(name, run->output_name) || (int32_t)dtype != run->output_dtype || rank != run->rank || !data ||
        bytes > lane->capacity || shape[0] != 1 || shape[rank - 1] != run->output_last) {
        lane->mismatch = 1;
        return VX_STATUS_INVALID_ARGUMENT;
    }
    for (uint32_t a = 1; a + 1 < rank; a++)
        if (shape[a] != run->input_shape[a]) lane->mismatch = 1;
    memcpy(lane->dst, data, bytes);
    lane->bytes = bytes;
    return lane->mismatch ? VX_STATUS_INVALID_ARGUMENT : VX_STATUS_OK;
}

int32_t mock_host_run_batch(MockRun* run, int32_t with_proof) {
    static const char fingerprint[] = "sha256:mock-graph-fingerprint";
    static const char proof[] = "sha256:mock-shape-domain-proof";
    static const char batch_proof[] = "sha256:mock-independent-batch-proof";
    VxRuntimeOptions runtime_options = VX_RUNTIME_OPTIONS_INIT;
    VxContextOptions context_options = VX_CONTEXT_OPTIONS_INIT;
    VxReport report = VX_REPORT_INIT;
    VxModelSource source = VX_MODEL_SOURCE_INIT;
    VxBackendCompileInput input = VX_BACKEND_COMPILE_INPUT_INIT;
    VxBackendShapeDomainAttestation attestation = VX_BACKEND_SHAPE_DOMAIN_ATTESTATION_INIT;
    VxBackendBatchContract contract = VX_BACKEND_BATCH_CONTRACT_INIT;
    VxBackendBatchInvocation invocation = VX_BACKEND_BATCH_INVOCATION_INIT;
    VxBackendPolicy policy = VX_BACKEND_POLICY_INIT;
    VxTensorSpec in_spec, out_spec;
    VxTensorBinding binding = VX_TENSOR_BINDING_INIT;
    const char* weights[1];
    const char* wanted[1];
    void *runtime = NULL, *compiled = NULL, *context = NULL;
    const uint32_t batch = (uint32_t)run->input_shape[0];
    VxBackendOutputSink* sinks = NULL;
    Lane* lanes = NULL;
    uint64_t* ids = NULL;
    VxStatus status;
    if (!g_registered || !g_provider.compiled_batch_contract || !g_provider.context_execute_batch || !batch)
        return run->status = VX_STATUS_BACKEND_UNSUPPORTED;
    status = g_provider.runtime_create(g_provider.user_data, &runtime_options, &runtime, &report);
    run->failed_stage = VX_STAGE_RUNTIME_CREATE;
    if (status != VX_STATUS_OK) goto done;
    weights[0] = run->weight_path;
    source.graph_path = run->graph_path;
    source.weight_paths = weights;
    source.weight_path_count = 1;
    spec_from(&in_spec, run->input_name, run->input_dtype, run, run->input_shape[run->rank - 1]);
    spec_from(&out_spec, run->output_name, run->output_dtype, run, run->output_last);
    input.source = &source;
    input.graph_fingerprint = fingerprint;
    input.shape_domain_proof_identity = proof;
    input.inputs = &in_spec;
    input.input_count = 1;
    input.outputs = &out_spec;
    input.output_count = 1;
    input.packed_arithmetic = (VxPackedArithmetic)run->packed_arithmetic;
    if (with_proof) {
        input.independent_batch_proof_protocol = VX_BACKEND_INDEPENDENT_BATCH_PROOF_PROTOCOL;
        input.independent_batch_proof_identity = batch_proof;
    }
    wanted[0] = g_name;
    policy.mode = VX_BACKEND_REQUIRE;
    policy.operator_fallback = VX_OPERATOR_FALLBACK_FORBID;
    policy.backends = wanted;
    policy.backend_count = 1;
    status = g_provider.compile(runtime, &input, &policy, &compiled, &attestation, &report);
    run->failed_stage = VX_STAGE_COMPILE;
    if (status != VX_STATUS_OK) goto done;
    status = g_provider.compiled_batch_contract(compiled, &contract, &report);
    if (status == VX_STATUS_OK &&
        (contract.struct_size != sizeof(contract) || !contract.protocol ||
         strcmp(contract.protocol, VX_BACKEND_BATCH_PROTOCOL) || !contract.resource_domain ||
         !contract.compatibility_token || !contract.min_batch || contract.max_batch < contract.min_batch ||
         !contract.multiple_of || contract.min_batch % contract.multiple_of || contract.batch_axis < 0 ||
         (contract.device_resident != 0 && contract.device_resident != 1)))
        status = VX_STATUS_ABI_UNSUPPORTED;
    if (status == VX_STATUS_OK && contract.max_batch > 1u &&
        (!with_proof || !contract.graph_fingerprint || strcmp(contract.graph_fingerprint, fingerprint) ||
         !contract.independent_batch_proof_identity || strcmp(contract.independent_batch_proof_identity, batch_proof) ||
         contract.batch_axis != 0 || (int64_t)contract.max_batch > run->lead_max[0]))
        status = VX_STATUS_ABI_UNSUPPORTED;
    run->attested_arithmetic = (int32_t)contract.max_batch; /* reported back: the frozen maximum */
    if (status != VX_STATUS_OK) goto done;
    if (batch > contract.max_batch) {
        status = VX_STATUS_BACKEND_UNSUPPORTED; /* the scheduler would not coalesce beyond the contract */
        goto done;
    }
    status = g_provider.context_create(compiled, &context_options, &context, &report);
    run->failed_stage = VX_STAGE_CONTEXT_CREATE;
    if (status != VX_STATUS_OK) goto done;

    sinks = (VxBackendOutputSink*)calloc(batch, sizeof(*sinks));
    lanes = (Lane*)calloc(batch, sizeof(*lanes));
    ids = (uint64_t*)calloc(batch, sizeof(*ids));
    for (uint32_t i = 0; i < batch; i++) {
        lanes[i].run = run;
        lanes[i].capacity = (size_t)(run->output_capacity / batch);
        lanes[i].dst = (unsigned char*)run->output + (size_t)i * lanes[i].capacity;
        sinks[i].struct_size = sizeof(sinks[i]);
        sinks[i].user_data = &lanes[i];
        sinks[i].write = lane_write;
        ids[i] = 1000u + i;
    }
    binding.name = run->input_name;
    binding.dtype = (VxDataType)run->input_dtype;
    binding.rank = run->rank;
    memcpy(binding.shape, run->input_shape, sizeof(binding.shape));
    binding.data = run->input;
    binding.byte_size = (size_t)run->input_bytes;
    binding.location = VX_MEMORY_HOST;
    invocation.stacked_inputs = &binding;
    invocation.stacked_input_count = 1;
    invocation.batch_size = batch;
    invocation.request_ids = ids;
    invocation.lane_output_sinks = sinks;
    invocation.lane_output_sink_count = batch;
    report = (VxReport)VX_REPORT_INIT;
    status = g_provider.context_execute_batch(context, &invocation, &report);
    run->failed_stage = VX_STAGE_EXECUTE;
    run->writes = 0;
    for (uint32_t i = 0; i < batch && status == VX_STATUS_OK; i++) {
        if (lanes[i].writes != 1 || lanes[i].mismatch || lanes[i].bytes != lanes[i].capacity) status = VX_STATUS_EXECUTION_FAILED;
        run->writes += lanes[i].writes;
    }
    run->execute_attested = report.route_attested && report.route_evidence[0];
    snprintf(run->execute_route, sizeof(run->execute_route), "%s", report.route_evidence);
    if (status == VX_STATUS_OK) run->failed_stage = VX_STAGE_NONE;
done:
    snprintf(run->message, sizeof(run->message), "%s", report.message);
    free(sinks);
    free(lanes);
    free(ids);
    if (context) g_provider.context_destroy(context);
    if (compiled) g_provider.compiled_destroy(compiled);
    if (runtime) g_provider.runtime_destroy(runtime);
    return run->status = status;
}

/* Row decode through the decode callbacks (native/include/volvoxai_backend.h:214-232), the way the
 * reference's Generate loop drives a provider context created with decode rows enabled
 * (native/src/runtime/public_api_execute_result.inc:563-576): one prefill at the last prompt
 * position, then one step per new token, the host feeding each step's ids back into the id rows.
 * Also holds the provider to the state rules: a step that is not at the next position is refused
 * and changes nothing; after a reset the same prefill gives the same ids. */
typedef struct MockDecode {
    /* in */
    const char* graph_path;
    const char* weight_path;
    const char* input_name;
    const char* ids_name;
    const char* logits_name; /* NULL: the graph declares the ids only */
    int32_t slots, capacity, vocab, prompt_len, steps;
    int32_t* token_ids;   /* [slots, capacity]: the prompt, generated ids are written behind it */
    int32_t* generated;   /* out [steps + 1, slots] */
    float* first_logits;  /* out [slots, vocab] when logits_name is set */
    /* out */
    int32_t status, failed_stage, writes, sink_mismatch;
    int32_t wrong_step_refused, reset_repeats, attested;
    char message[VX_REPORT_MESSAGE_CAPACITY];
    char compile_route[VX_REPORT_ROUTE_CAPACITY];
    char execute_route[VX_REPORT_ROUTE_CAPACITY];
    int32_t replayed_steps; /* steps whose route evidence says they were a replay of the recorded step */
    double step_seconds;    /* wall time of the steps after the second (those that can be replays), summed */
} MockDecode;

typedef struct DecodeSink {
    MockDecode* run;
    int32_t* ids;
    float* logits;
    int32_t ids_written, logits_written;
} DecodeSink;

static VxStatus decode_write(void* user, const char* name, VxDataType dtype, const int64_t* shape, uint32_t rank,
                             const void* data, size_t bytes) {
    DecodeSink* sink = (DecodeSink*)user;
    MockDecode* run = sink->run;
    run->writes++;
    if (name && !strcmp(name, run->ids_name) && dtype == VX_DTYPE_I32 && rank == 1 && shape[0] == run->slots && data &&
        bytes == (size_t)run->slots * 4u && !sink->ids_written) {
        memcpy(sink->ids, data, bytes);
        sink->ids_written = 1;
        return VX_STATUS_OK;
    }
    if (name && run->logits_name && !strcmp(name, run->logits_name) && dtype == VX_DTYPE_F32 && rank == 2 &&
        shape[0] == run->slots && shape[1] == run->vocab && data && bytes == (size_t)run->slots * run->vocab * 4u &&
        !sink->logits_written) {
        if (sink->logits) memcpy(sink->logits, data, bytes);
        sink->logits_written = 1;
        return VX_STATUS_OK;
    }
    run->sink_mismatch = 1;
    return VX_STATUS_INVALID_ARGUMENT;
}

static void fixed_spec(VxTensorSpec* spec, const char* name, VxDataType dtype, uint32_t rank, int64_t d0, int64_t d1) {
    memset(spec, 0, sizeof(*spec));
    spec->struct_size = sizeof(*spec);
    spec->name = name;
    spec->dtype = dtype;
    spec->rank = rank;
    spec->location = VX_MEMORY_HOST;
    for (uint32_t a = 0; a < rank; a++) {
        VxDimensionConstraint* d = &spec->dimensions[a];
        d->struct_size = sizeof(*d);
        d->kind = VX_DIMENSION_FIXED;
        d->multiple_of = 1;
        d->min = d->max = a ? d1 : d0;
    }
}

int32_t mock_host_run_decode(MockDecode* run) {
    static const char fingerprint[] = "sha256:mock-graph-fingerprint";
    static const char proof[] = "sha256:mock-shape-domain-proof";
    VxRuntimeOptions runtime_options = VX_RUNTIME_OPTIONS_INIT;
    VxContextOptions context_options = VX_CONTEXT_OPTIONS_INIT;
    VxReport report = VX_REPORT_INIT;
    VxModelSource source = VX_MODEL_SOURCE_INIT;
    VxBackendCompileInput input = VX_BACKEND_COMPILE_INPUT_INIT;
    VxBackendShapeDomainAttestation attestation = VX_BACKEND_SHAPE_DOMAIN_ATTESTATION_INIT;
    VxBackendPolicy policy = VX_BACKEND_POLICY_INIT;
    VxTensorSpec in_spec, out_specs[2];
    VxTensorBinding binding = VX_TENSOR_BINDING_INIT;
    DecodeSink state = {run, NULL, NULL, 0, 0};
    VxBackendOutputSink sink = {sizeof(VxBackendOutputSink), &state, decode_write};
    const char* weights[1];
    const char* wanted[1];
    const char* decode_inputs[1];
    void *runtime = NULL, *compiled = NULL, *context = NULL;
    int32_t* again = NULL;
    const int32_t expected_writes = run->logits_name ? 2 : 1;
    VxStatus status;
    if (!g_registered) return run->status = VX_STATUS_NOT_FOUND;
    if (!g_provider.context_decode_prefill || !g_provider.context_decode_step || !g_provider.context_decode_reset)
        return run->status = VX_STATUS_BACKEND_UNSUPPORTED;
    run->writes = run->sink_mismatch = run->wrong_step_refused = run->reset_repeats = run->attested = run->replayed_steps = 0;
    run->step_seconds = 0.0;
    status = g_provider.runtime_create(g_provider.user_data, &runtime_options, &runtime, &report);
    run->failed_stage = VX_STAGE_RUNTIME_CREATE;
    if (status != VX_STATUS_OK) goto done;
    weights[0] = run->weight_path;
    source.graph_path = run->graph_path;
    source.weight_paths = weights;
    source.weight_path_count = 1;
    fixed_spec(&in_spec, run->input_name, VX_DTYPE_I32, 2, run->slots, run->capacity);
    fixed_spec(&out_specs[0], run->ids_name, VX_DTYPE_I32, 1, run->slots, 0);
    if (run->logits_name) fixed_spec(&out_specs[1], run->logits_name, VX_DTYPE_F32, 2, run->slots, run->vocab);
    input.source = &source;
    input.graph_fingerprint = fingerprint;
    input.shape_domain_proof_identity = proof;
    input.inputs = &in_spec;
    input.input_count = 1;
    input.outputs = out_specs;
    input.output_count = (size_t)expected_writes;
    input.packed_arithmetic = VX_PACKED_ARITHMETIC_DYNAMIC_I8;
    wanted[0] = g_name;
    policy.mode = VX_BACKEND_REQUIRE;
    policy.operator_fallback = VX_OPERATOR_FALLBACK_FORBID;
    policy.backends = wanted;
    policy.backend_count = 1;
    report = (VxReport)VX_REPORT_INIT;
    status = g_provider.compile(runtime, &input, &policy, &compiled, &attestation, &report);
    run->failed_stage = VX_STAGE_COMPILE;
    if (status != VX_STATUS_OK) {
        if (compiled) status = VX_STATUS_INTERNAL;
        goto done;
    }
    snprintf(run->compile_route, sizeof(run->compile_route), "%s", report.route_evidence);
    run->attested = report.route_attested && !report.operator_fallback_used && attestation.graph_fingerprint &&
                    !strcmp(attestation.graph_fingerprint, fingerprint) &&
                    attestation.packed_arithmetic == VX_PACKED_ARITHMETIC_DYNAMIC_I8;

    decode_inputs[0] = run->input_name;
    context_options.decode_row_mode = VX_DECODE_ROW_REQUIRED;
    context_options.require_incremental = 1;
    context_options.decode_slots = (uint32_t)run->slots;
    context_options.decode_inputs = decode_inputs;
    context_options.decode_input_count = 1;
    report = (VxReport)VX_REPORT_INIT;
    status = g_provider.context_create(compiled, &context_options, &context, &report);
    run->failed_stage = VX_STAGE_CONTEXT_CREATE;
    if (status != VX_STATUS_OK) goto done;

    binding.name = run->input_name;
    binding.dtype = VX_DTYPE_I32;
    binding.rank = 2;
    binding.shape[0] = run->slots;
    binding.shape[1] = run->capacity;
    binding.data = run->token_ids;
    binding.byte_size = (size_t)run->slots * run->capacity * 4u;
    binding.location = VX_MEMORY_HOST;
    run->failed_stage = VX_STAGE_EXECUTE;

    /* prefill: rows 0 .. prompt_len-1 */
    state.ids = run->generated;
    state.logits = run->first_logits;
    report = (VxReport)VX_REPORT_INIT;
    status = g_provider.context_decode_prefill(context, run->prompt_len - 1, &binding, 1, &sink, &report);
    if (status == VX_STATUS_OK && (run->writes != expected_writes || run->sink_mismatch)) status = VX_STATUS_EXECUTION_FAILED;
    if (status != VX_STATUS_OK) goto done;
    run->attested = run->attested && report.route_attested && report.route_evidence[0];
    snprintf(run->execute_route, sizeof(run->execute_route), "%s", report.route_evidence);
    /* a step that skips a position is refused and leaves the state alone */
    {
        DecodeSink scratch_state = {run, (int32_t*)calloc((size_t)run->slots, 4u), NULL, 0, 0};
        VxBackendOutputSink scratch = {sizeof(VxBackendOutputSink), &scratch_state, decode_write};
        const int32_t before = run->writes;
        VxReport r2 = VX_REPORT_INIT;
        VxStatus refused = g_provider.context_decode_step(context, run->prompt_len + 1, &binding, 1, &scratch, &r2);
        run->wrong_step_refused = refused == VX_STATUS_INVALID_ARGUMENT && run->writes == before;
        free(scratch_state.ids);
    }
    for (int32_t i = 1; i <= run->steps && status == VX_STATUS_OK; i++) {
        const int32_t position = run->prompt_len + i - 1; /* the column of the token generated last */
        const int32_t before = run->writes;
        if (position >= run->capacity) {
            status = VX_STATUS_INVALID_ARGUMENT;
            break;
        }
        for (int32_t r = 0; r < run->slots; r++)
            run->token_ids[(size_t)r * run->capacity + position] = run->generated[(size_t)(i - 1) * run->slots + r];
        state.ids = run->generated + (size_t)i * run->slots;
        state.logits = NULL;
        state.ids_written = state.logits_written = 0;
        report = (VxReport)VX_REPORT_INIT;
        {
            struct timespec t0, t1;
            clock_gettime(CLOCK_MONOTONIC, &t0);
            status = g_provider.context_decode_step(context, position, &binding, 1, &sink, &report);
            clock_gettime(CLOCK_MONOTONIC, &t1);
            if (i > 2) run->step_seconds += (double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec);
        }
        if (status == VX_STATUS_OK && (run->writes != before + expected_writes || run->sink_mismatch))
            status = VX_STATUS_EXECUTION_FAILED;
        if (status == VX_STATUS_OK && strstr(report.route_evidence, "+replay")) run->replayed_steps++;
    }
    if (status != VX_STATUS_OK) goto done;
    /* reset, then the same prefill again: the same first ids */
    again = (int32_t*)calloc((size_t)run->slots, 4u);
    report = (VxReport)VX_REPORT_INIT;
    status = g_provider.context_decode_reset(context, &report);
    if (status == VX_STATUS_OK) {
        state.ids = again;
        state.logits = NULL;
        state.ids_written = state.logits_written = 0;
        report = (VxReport)VX_REPORT_INIT;
        status = g_provider.context_decode_prefill(context, run->prompt_len - 1, &binding, 1, &sink, &report);
        run->reset_repeats = status == VX_STATUS_OK && !memcmp(again, run->generated, (size_t)run->slots * 4u);
    }
    if (status == VX_STATUS_OK) run->failed_stage = VX_STAGE_NONE;
done:
    snprintf(run->message, sizeof(run->message), "%s", report.message);
    free(again);
    if (context) {
        if (g_provider.context_close) (void)g_provider.context_close(context, &report);
        g_provider.context_destroy(context);
    }
    if (compiled) g_provider.compiled_destroy(compiled);
    if (runtime) g_provider.runtime_destroy(runtime);
    return run->status = status;
}

/* A graph with several inputs and outputs: every input bound by name in one context_execute (or
 * one context_execute_batch over `batch` lanes stacked along axis 0), every declared output
 * written exactly once (per lane) with its own name, dtype and shape. */
typedef struct MockPort {
    const char* name;
    int32_t dtype;
    int64_t last; /* last extent */
    void* data;   /* input bytes, or the buffer an output is copied into */
    uint64_t bytes;
    int32_t written;
} MockPort;

typedef struct MockGraphRun {
    /* in */
    const char* graph_path;
    const char* weight_path;
    int32_t packed_arithmetic;
    uint32_t rank;
    int64_t lead[VX_MAX_TENSOR_RANK]; /* the leading extents of every tensor */
    int64_t lead_max0;                /* > 0: axis 0 is symbolic, bounded 1..lead_max0 */
    int32_t batch;                    /* > 0: run as one scheduler batch of lead[0] lanes */
    int32_t input_count, output_count;
    MockPort inputs[8], outputs[8];
    /* out */
    int32_t status, failed_stage, writes, sink_mismatch;
    char message[VX_REPORT_MESSAGE_CAPACITY];
    char execute_route[VX_REPORT_ROUTE_CAPACITY];
} MockGraphRun;

typedef struct GraphLane {
    MockGraphRun* run;
    int32_t lane; /* -1: the whole tensor */
    int32_t written[8];
} GraphLane;

static VxStatus graph_write(void* user, const char* name, VxDataType dtype, const int64_t* shape, uint32_t rank,
                            const void* data, size_t bytes) {
    GraphLane* lane = (GraphLane*)user;
    MockGraphRun* run = lane->run;
    run->writes++;
    for (int32_t k = 0; name && k < run->output_count; k++) {
        MockPort* port = &run->outputs[k];
        const size_t lanes = lane->lane < 0 ? 1u : (size_t)run->lead[0];
        int ok = !strcmp(name, port->name) && (int32_t)dtype == port->dtype && rank == run->rank && data &&
                 bytes == (size_t)port->bytes / lanes && shape[rank - 1] == port->last && !lane->written[k];
        if (strcmp(name, port->name)) continue;
        for (uint32_t a = 0; ok && a + 1 < rank; a++)
            if (shape[a] != (a == 0 && lane->lane >= 0 ? 1 : run->lead[a])) ok = 0;
        if (!ok) break;
        memcpy((unsigned char*)port->data + (lane->lane < 0 ? 0u : (size_t)lane->lane * bytes), data, bytes);
        lane->written[k] = 1;
        port->written++;
        return VX_STATUS_OK;
    }
    run->sink_mismatch = 1;
    return VX_STATUS_INVALID_ARGUMENT;
}

static void port_spec(VxTensorSpec* spec, const MockGraphRun* run, const MockPort* port) {
    memset(spec, 0, sizeof(*spec));
    spec->struct_size = sizeof(*spec);
    spec->name = port->name;
    spec->dtype = (VxDataType)port->dtype;
    spec->rank = run->rank;
    spec->location = VX_MEMORY_HOST;
    for (uint32_t a = 0; a < run->rank; a++) {
        VxDimensionConstraint* d = &spec->dimensions[a];
        d->struct_size = sizeof(*d);
        d->multiple_of = 1;
        if (a == 0 && run->rank > 1 && run->lead_max0 > 0) {
            d->kind = VX_DIMENSION_SYMBOLIC;
            d->symbol = "rows";
            d->min = 1;
            d->max = run->lead_max0;
        } else {
            d->kind = VX_DIMENSION_FIXED;
            d->min = d->max = a + 1 < run->rank ? run->lead[a] : port->last;
        }
    }
}

int32_t mock_host_run_graph(MockGraphRun* run) {
    static const char fingerprint[] = "sha256:mock-graph-fingerprint";
    static const char proof[] = "sha256:mock-shape-domain-proof";
    static const char batch_proof[] = "sha256:mock-independent-batch-proof";
    VxRuntimeOptions runtime_options = VX_RUNTIME_OPTIONS_INIT;
    VxContextOptions context_options = VX_CONTEXT_OPTIONS_INIT;
    VxReport report = VX_REPORT_INIT;
    VxModelSource source = VX_MODEL_SOURCE_INIT;
    VxBackendCompileInput input = VX_BACKEND_COMPILE_INPUT_INIT;
    VxBackendShapeDomainAttestation attestation = VX_BACKEND_SHAPE_DOMAIN_ATTESTATION_INIT;
    VxBackendPolicy policy = VX_BACKEND_POLICY_INIT;
    VxTensorSpec in_specs[8], out_specs[8];
    VxTensorBinding bindings[8];
    const char* weights[1];
    const char* wanted[1];
    void *runtime = NULL, *compiled = NULL, *context = NULL;
    VxStatus status;
    if (!g_registered || run->input_count < 1 || run->input_count > 8 || run->output_count < 1 || run->output_count > 8)
        return run->status = VX_STATUS_INVALID_ARGUMENT;
    run->writes = run->sink_mismatch = 0;
    for (int32_t k = 0; k < run->output_count; k++) run->outputs[k].written = 0;
    status = g_provider.runtime_create(g_provider.user_data, &runtime_options, &runtime, &report);
    run->failed_stage = VX_STAGE_RUNTIME_CREATE;
    if (status != VX_STATUS_OK) goto done;
    weights[0] = run->weight_path;
    source.graph_path = run->graph_path;
    source.weight_paths = weights;
    source.weight_path_count = 1;
    for (int32_t k = 0; k < run->input_count; k++) port_spec(&in_specs[k], run, &run->inputs[k]);
    for (int32_t k = 0; k < run->output_count; k++) port_spec(&out_specs[k], run, &run->outputs[k]);
    input.source = &source;
    input.graph_fingerprint = fingerprint;
    input.shape_domain_proof_identity = proof;
    input.inputs = in_specs;
    input.input_count = (size_t)run->input_count;
    input.outputs = out_specs;
    input.output_count = (size_t)run->output_count;
    input.packed_arithmetic = (VxPackedArithmetic)run->packed_arithmetic;
    if (run->batch > 0) {
        input.independent_batch_proof_protocol = VX_BACKEND_INDEPENDENT_BATCH_PROOF_PROTOCOL;
        input.independent_batch_proof_identity = batch_proof;
    }
    wanted[0] = g_name;
    policy.mode = VX_BACKEND_REQUIRE;
    policy.operator_fallback = VX_OPERATOR_FALLBACK_FORBID;
    policy.backends = wanted;
    policy.backend_count = 1;
    report = (VxReport)VX_REPORT_INIT;
    status = g_provider.compile(runtime, &input, &policy, &compiled, &attestation, &report);
    run->failed_stage = VX_STAGE_COMPILE;
    if (status != VX_STATUS_OK) {
        if (compiled) status = VX_STATUS_INTERNAL;
        goto done;
    }
    report = (VxReport)VX_REPORT_INIT;
    status = g_provider.context_create(compiled, &context_options, &context, &report);
    run->failed_stage = VX_STAGE_CONTEXT_CREATE;
    if (status != VX_STATUS_OK) goto done;
    /* the bindings in reverse order of the declaration: a provider finds them by name */
    for (int32_t k = 0; k < run->input_count; k++) {
        VxTensorBinding* b = &bindings[run->input_count - 1 - k];
        *b = (VxTensorBinding)VX_TENSOR_BINDING_INIT;
        b->name = run->inputs[k].name;
        b->dtype = (VxDataType)run->inputs[k].dtype;
        b->rank = run->rank;
        for (uint32_t a = 0; a + 1 < run->rank; a++) b->shape[a] = run->lead[a];
        b->shape[run->rank - 1] = run->inputs[k].last;
        b->data = run->inputs[k].data;
        b->byte_size = (size_t)run->inputs[k].bytes;
        b->location = VX_MEMORY_HOST;
    }
    run->failed_stage = VX_STAGE_EXECUTE;
    report = (VxReport)VX_REPORT_INIT;
    if (run->batch > 0) {
        const uint32_t batch = (uint32_t)run->lead[0];
        VxBackendBatchContract contract = VX_BACKEND_BATCH_CONTRACT_INIT;
        VxBackendBatchInvocation invocation = VX_BACKEND_BATCH_INVOCATION_INIT;
        VxBackendOutputSink* sinks = (VxBackendOutputSink*)calloc(batch, sizeof(*sinks));
        GraphLane* lanes = (GraphLane*)calloc(batch, sizeof(*lanes));
        status = g_provider.compiled_batch_contract(compiled, &contract, &report);
        if (status == VX_STATUS_OK && batch > contract.max_batch) status = VX_STATUS_BACKEND_UNSUPPORTED;
        for (uint32_t i = 0; i < batch; i++) {
            lanes[i].run = run;
            lanes[i].lane = (int32_t)i;
            sinks[i].struct_size = sizeof(sinks[i]);
            sinks[i].user_data = &lanes[i];
            sinks[i].write = graph_write;
        }
        invocation.stacked_inputs = bindings;
        invocation.stacked_input_count = (size_t)run->input_count;
        invocation.batch_size = batch;
        invocation.lane_output_sinks = sinks;
        invocation.lane_output_sink_count = batch;
        report = (VxReport)VX_REPORT_INIT;
        if (status == VX_STATUS_OK) status = g_provider.context_execute_batch(context, &invocation, &report);
        for (int32_t k = 0; status == VX_STATUS_OK && k < run->output_count; k++)
            if (run->outputs[k].written != (int32_t)batch) status = VX_STATUS_EXECUTION_FAILED;
        free(sinks);
        free(lanes);
    } else {
        GraphLane whole = {run, -1, {0}};
        VxBackendOutputSink sink = {sizeof(VxBackendOutputSink), &whole, graph_write};
        status = g_provider.context_execute(context, bindings, (size_t)run->input_count, &sink, &report);
        for (int32_t k = 0; status == VX_STATUS_OK && k < run->output_count; k++)
            if (run->outputs[k].written != 1) status = VX_STATUS_EXECUTION_FAILED;
    }
    if (status == VX_STATUS_OK && run->sink_mismatch) status = VX_STATUS_EXECUTION_FAILED;
    snprintf(run->execute_route, sizeof(run->execute_route), "%s", report.route_evidence);
    if (status == VX_STATUS_OK) run->failed_stage = VX_STAGE_NONE;
done:
    snprintf(run->message, sizeof(run->message), "%s", report.message);
    if (context) {
        if (g_provider.context_close) (void)g_provider.context_close(context, &report);
        g_provider.context_destroy(context);
    }
    if (compiled) g_provider.compiled_destroy(compiled);
    if (runtime) g_provider.runtime_destroy(runtime);
    return run->status = status;
}
