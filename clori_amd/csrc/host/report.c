/*
 * Backend reports, their text rendering and the two inspection commands of the ROCm arm:
 * `inspect backend rocm` and `inspect rocm [bandwidth]`.
 *
 * The split follows the reference: a typed report is built from backend facts
 * (src/backend/core.c:1824-1916), a renderer turns the report into text without deciding
 * anything (src/cli/render/backend.c:51-160), and the command maps the report's exit code
 * (src/cli/commands/backend.c:11-52).  Opening a backend that is not usable here is not an
 * error of the command: the report says "unsupported", carries the reason and exit code 5
 * (tests/test_cuda_failclosed.sh:46-57).
 *
 * Also here: the sample summary of a component benchmark
 * (src/runtime/benchmark.c:388-447), so that a benchmark record of this backend carries the
 * same distribution, by the same rule, as the reference's records.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "private.h"

const char *yvex_backend_bundle_admission_name(yvex_backend_bundle_admission admission)
{
    switch (admission) {
    case YVEX_BACKEND_BUNDLE_NOT_APPLICABLE: return "not-applicable";
    case YVEX_BACKEND_BUNDLE_ABSENT: return "absent";
    case YVEX_BACKEND_BUNDLE_ADMITTED: return "admitted";
    case YVEX_BACKEND_BUNDLE_REJECTED: return "rejected";
    }
    return "rejected";
}

static int report_fail(yvex_backend *backend, int rc)
{
    yvex_backend_close(backend);
    return rc;
}

int yvex_backend_report_build(const yvex_backend_report_request *request,
                              yvex_backend_report *report, yvex_error *err)
{
    static const yvex_backend_operation_variant rocm_variants[] = {
        YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_F32,  YVEX_BACKEND_VARIANT_ROCM_ATTENTION_GQA_BF16,
        YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_BF16, YVEX_BACKEND_VARIANT_ROCM_ATTENTION_PAGED_Q8_0,
        YVEX_BACKEND_VARIANT_ROCM_ATTENTION_MLA_BF16,
    };
    yvex_backend *backend = NULL;
    yvex_backend_options options;
    yvex_backend_rocm_report rocm;
    unsigned int i;
    int rocm_kind, rc;

    if (!request || !report) {
        yvex_error_set(err, YVEX_ERR_INVALID_ARG, "yvex_backend_report_build",
                       "request and report are required");
        return YVEX_ERR_INVALID_ARG;
    }
    rocm_kind = request->kind == YVEX_BACKEND_REPORT_ROCM_INFO ||
                request->kind == YVEX_BACKEND_REPORT_ROCM_BANDWIDTH;
    if ((request->kind != YVEX_BACKEND_REPORT_CAPABILITIES && !rocm_kind) ||
        (rocm_kind && request->backend_kind != YVEX_BACKEND_KIND_ROCM)) {
        yvex_error_set(err, YVEX_ERR_INVALID_ARG, "yvex_backend_report_build",
                       "request and report are required");
        return YVEX_ERR_INVALID_ARG;
    }
    memset(report, 0, sizeof(*report));
    memset(&options, 0, sizeof(options));
    report->kind = request->kind;
    report->backend_kind = request->backend_kind;
    report->backend_status = YVEX_BACKEND_STATUS_UNSUPPORTED;
    report->bundle_admission = YVEX_BACKEND_BUNDLE_NOT_APPLICABLE;
    options.kind = request->backend_kind;

    rc = yvex_backend_open(&backend, &options, err);
    if (rc == YVEX_ERR_UNSUPPORTED) {
        report->exit_code = 5;
        snprintf(report->reason, sizeof(report->reason), "%s",
                 err && err->message[0] ? err->message : "backend unavailable");
        yvex_error_clear(err);
        return YVEX_OK;
    }
    if (rc != YVEX_OK) return rc;

    report->available = 1;
    report->backend_status = yvex_backend_status_of(backend);
    rc = yvex_backend_get_memory_stats(backend, &report->memory, err);
    if (rc == YVEX_OK) rc = yvex_backend_get_device_info(backend, &report->device_info, err);
    if (rc != YVEX_OK) return report_fail(backend, rc);
    report->has_device_info = 1;
    snprintf(report->device_name, sizeof(report->device_name), "%s",
             report->device_info.name ? report->device_info.name : "");
    report->device_info.name = report->device_name;

    for (i = 0; i <= (unsigned int)YVEX_BACKEND_CAP_OP_ATTENTION; ++i)
        report->capabilities[i] = yvex_backend_supports(backend, (yvex_backend_capability)i);
    if (request->backend_kind == YVEX_BACKEND_KIND_ROCM) {
        const yvex_backend_capability_result *first;
        for (i = 0; i < (unsigned int)YVEX_BACKEND_VARIANT_COUNT; ++i) {
            rc = yvex_backend_query_capability(backend, (yvex_backend_operation_variant)i,
                                               &report->variants[report->variant_count++], err);
            if (rc != YVEX_OK) return report_fail(backend, rc);
        }
        for (i = 0; i < sizeof(rocm_variants) / sizeof(rocm_variants[0]); ++i) {
            rc = yvex_backend_query_capability(backend, rocm_variants[i],
                                               &report->variants[report->variant_count++], err);
            if (rc != YVEX_OK) return report_fail(backend, rc);
        }
        /* bundle admission is read off one bundle-backed variant, as the reference reads it
         * off the embed variant (src/backend/core.c:1808-1822) */
        first = &report->variants[YVEX_BACKEND_VARIANT_COUNT];
        report->context_available = (unsigned int)first->context_available;
        report->bundle_reason = first->reason;
        if (first->kernel_bundle_available)
            report->bundle_admission = YVEX_BACKEND_BUNDLE_ADMITTED;
        else if (first->reason == YVEX_BACKEND_CAPABILITY_REASON_KERNEL_BUNDLE_ABSENT)
            report->bundle_admission = YVEX_BACKEND_BUNDLE_ABSENT;
        else
            report->bundle_admission = YVEX_BACKEND_BUNDLE_REJECTED;
        rc = yvex_backend_rocm_report_get(backend, &rocm, err);
        if (rc != YVEX_OK) return report_fail(backend, rc);
        /* every image of the bundle is built for one ISA and nothing is translated at load */
        report->kernel_bundle_native = rocm.bundle_admitted;
        yvex_core_text_copy(report->kernel_bundle_architecture,
                            sizeof(report->kernel_bundle_architecture), rocm.architecture);
        report->kernel_image_count = rocm.image_count;
        report->kernel_function_count = rocm.function_count;
        yvex_core_text_copy(report->driver_library, sizeof(report->driver_library),
                            rocm.driver_library);
        if (request->kind == YVEX_BACKEND_REPORT_ROCM_BANDWIDTH) {
            rc = yvex_backend_bandwidth_probe(backend, &report->bandwidth, err);
            if (rc != YVEX_OK) return report_fail(backend, rc);
        }
    }
    yvex_backend_close(backend);
    yvex_error_clear(err);
    return YVEX_OK;
}

/* ---- rendering ------------------------------------------------------------------------ */

static const char *yes_no(int value)
{
    return value ? "yes" : "no";
}

static void render_admission(FILE *fp, const yvex_backend_report *report)
{
    fprintf(fp, "context_available: %s\n", yes_no((int)report->context_available));
    fprintf(fp, "kernel_bundle: %s\n", yvex_backend_bundle_admission_name(report->bundle_admission));
    fprintf(fp, "kernel_bundle_reason: %s\n",
            yvex_backend_capability_reason_name(report->bundle_reason));
    fprintf(fp, "kernel_bundle_native: %s\n", yes_no(report->kernel_bundle_native));
    fprintf(fp, "kernel_bundle_architecture: %s\n",
            report->kernel_bundle_architecture[0] ? report->kernel_bundle_architecture
                                                  : "unavailable");
    fprintf(fp, "kernel_bundle_identity: %s\n",
            report->kernel_bundle_identity[0] ? report->kernel_bundle_identity : "unavailable");
    fprintf(fp, "kernel_bundle_images: %u\nkernel_bundle_functions: %u\n",
            report->kernel_image_count, report->kernel_function_count);
}

static void render_capabilities(FILE *fp, const yvex_backend_report *report)
{
    unsigned int i;
    fprintf(fp, "backend: %s\n", yvex_backend_kind_name(report->backend_kind));
    if (!report->available) {
        fprintf(fp, "status: unsupported\nreason: %s\n", report->reason);
        fprintf(fp, "status: backend-unsupported\n");
        return;
    }
    fprintf(fp, "status: %s\n", yvex_backend_status_name(report->backend_status));
    if (report->backend_kind == YVEX_BACKEND_KIND_ROCM && report->has_device_info) {
        fprintf(fp, "device: %d\nname: %s\ncompute_capability: %d.%d\n",
                report->device_info.device_index, report->device_info.name,
                report->device_info.compute_capability_major,
                report->device_info.compute_capability_minor);
        fprintf(fp, "memory:\n  free_bytes: %llu\n  total_bytes: %llu\n",
                report->device_info.free_memory_bytes, report->device_info.total_memory_bytes);
    } else {
        fprintf(fp, "memory:\n");
    }
    fprintf(fp,
            "  allocated_bytes: %llu\n  allocation_count: %llu\n  peak_allocated_bytes: %llu\n"
            "capabilities:\n",
            report->memory.allocated_bytes, report->memory.allocation_count,
            report->memory.peak_allocated_bytes);
    for (i = 0; i <= (unsigned int)YVEX_BACKEND_CAP_OP_ATTENTION; ++i)
        fprintf(fp, "  %s: %s\n", yvex_backend_capability_name((yvex_backend_capability)i),
                yes_no(report->capabilities[i]));
    if (report->backend_kind == YVEX_BACKEND_KIND_ROCM) {
        render_admission(fp, report);
        fprintf(fp, "variants:\n");
        for (i = 0; i < report->variant_count; ++i) {
            const yvex_backend_capability_result *result = &report->variants[i];
            fprintf(fp, "  %s: %s (%s)\n", yvex_backend_operation_variant_name(result->variant),
                    yvex_backend_capability_state_name(result->state),
                    yvex_backend_capability_reason_name(result->reason));
        }
    }
    fprintf(fp, "status: backend-capabilities\n");
}

static void render_rocm_info(FILE *fp, const yvex_backend_report *report)
{
    if (!report->available) {
        fprintf(fp, "rocm: unavailable\nreason: %s\n", report->reason);
        fprintf(fp, "status: rocm-unavailable\n");
        return;
    }
    fprintf(fp, "rocm: available\ndevice_count: >=1\n\n");
    fprintf(fp,
            "device %d:\n  name: %s\n  compute_capability: %d.%d\n  global_memory_bytes: %llu\n"
            "  free_memory_bytes: %llu\n  total_memory_bytes: %llu\n  unified_addressing: %s\n"
            "  managed_memory: %s\n  driver_library: %s\n",
            report->device_info.device_index, report->device_info.name,
            report->device_info.compute_capability_major,
            report->device_info.compute_capability_minor, report->device_info.global_memory_bytes,
            report->device_info.free_memory_bytes, report->device_info.total_memory_bytes,
            yes_no(report->device_info.unified_addressing),
            yes_no(report->device_info.managed_memory),
            report->driver_library[0] ? report->driver_library : "unavailable");
    render_admission(fp, report);
    fprintf(fp, "\nstatus: rocm-info\n");
}

static void render_rocm_bandwidth(FILE *fp, const yvex_backend_report *report)
{
    const yvex_backend_bandwidth_evidence *evidence = &report->bandwidth;
    unsigned int index;
    if (!report->available) {
        render_rocm_info(fp, report);
        return;
    }
    fprintf(fp,
            "rocm_bandwidth_schema: %u\nworking_set_bytes: %llu\niterations: %llu\n"
            "sample_count: %llu\nkernel_bundle_identity: %s\nevidence_identity: %s\n"
            "sustainable_read_bytes_per_second: %llu\n"
            "sustainable_copy_bytes_per_second: %llu\n"
            "sustainable_coherent_host_bytes_per_second: %llu\nsamples:\n",
            evidence->schema_version, evidence->working_set_bytes, evidence->iterations,
            evidence->sample_count, evidence->kernel_bundle_identity, evidence->identity,
            evidence->sustainable_read_bytes_per_second,
            evidence->sustainable_copy_bytes_per_second,
            evidence->sustainable_coherent_host_bytes_per_second);
    for (index = 0u; index < evidence->sample_count; ++index)
        fprintf(fp, "  %u: stream_ns=%llu copy_ns=%llu coherent_host_ns=%llu\n", index + 1u,
                evidence->stream_elapsed_ns[index], evidence->copy_elapsed_ns[index],
                evidence->coherent_host_elapsed_ns[index]);
    fprintf(fp, "status: rocm-bandwidth\n");
}

int yvex_backend_render(void *stream, const yvex_backend_report *report)
{
    FILE *fp = stream;
    if (!fp || !report) return YVEX_ERR_INVALID_ARG;
    if (report->kind == YVEX_BACKEND_REPORT_ROCM_BANDWIDTH)
        render_rocm_bandwidth(fp, report);
    else if (report->kind == YVEX_BACKEND_REPORT_ROCM_INFO)
        render_rocm_info(fp, report);
    else
        render_capabilities(fp, report);
    return YVEX_OK;
}

/* ---- commands ------------------------------------------------------------------------- */

/* src/cli/io/out.c:1277-1292 */
static int exit_for_status(int status)
{
    switch (status) {
    case YVEX_ERR_INVALID_ARG: return 2;
    case YVEX_ERR_IO: return 3;
    case YVEX_ERR_FORMAT:
    case YVEX_ERR_BOUNDS: return 4;
    case YVEX_ERR_UNSUPPORTED: return 5;
    default: return 1;
    }
}

static int command_error(const yvex_error *err, int rc)
{
    fprintf(stderr, "yvex: %s: %s\n", err->where, err->message);
    return rc == YVEX_ERR_NOMEM ? 3 : exit_for_status(rc);
}

static int is_help(const char *argument)
{
    return strcmp(argument, "--help") == 0 || strcmp(argument, "-h") == 0;
}

static int command_run(const yvex_backend_report_request *request)
{
    yvex_backend_report *report = calloc(1u, sizeof(*report));
    yvex_error err;
    int rc;
    yvex_error_clear(&err);
    if (!report) {
        yvex_error_set(&err, YVEX_ERR_NOMEM, "backend", "report allocation failed");
        return command_error(&err, YVEX_ERR_NOMEM);
    }
    rc = yvex_backend_report_build(request, report, &err);
    if (rc != YVEX_OK) {
        free(report);
        return command_error(&err, rc);
    }
    (void)yvex_backend_render(stdout, report);
    fflush(stdout);
    rc = report->exit_code;
    free(report);
    return rc;
}

/* argv is the adapter's: {program, "backend", kind} (src/cli/input/backend.c:17-50). */
int yvex_backend_command(int argc, char **argv)
{
    yvex_backend_report_request request = {YVEX_BACKEND_REPORT_CAPABILITIES, YVEX_BACKEND_KIND_ROCM};
    yvex_error err;
    yvex_error_clear(&err);
    if (!argv) {
        yvex_error_set(&err, YVEX_ERR_INVALID_ARG, "backend", "backend arguments are required");
        return command_error(&err, YVEX_ERR_INVALID_ARG);
    }
    if (argc == 3 && is_help(argv[2])) {
        printf("usage: yvex inspect backend rocm\n\n"
               "Reports context, bundle, and exact primitive capabilities.\n");
        return 0;
    }
    if (argc != 3) {
        yvex_error_set(&err, YVEX_ERR_INVALID_ARG, "backend", "backend requires rocm");
        return command_error(&err, YVEX_ERR_INVALID_ARG);
    }
    if (yvex_backend_kind_parse(argv[2], &request.backend_kind, &err) != YVEX_OK) {
        yvex_error_setf(&err, YVEX_ERR_INVALID_ARG, "backend", "unknown backend kind: %s", argv[2]);
        return command_error(&err, YVEX_ERR_INVALID_ARG);
    }
    return command_run(&request);
}

/* argv is the adapter's: {program, "rocm-info"[, "bandwidth"]}
 * (src/cli/input/backend.c:52-85). */
int yvex_rocm_info_command(int argc, char **argv)
{
    yvex_backend_report_request request = {YVEX_BACKEND_REPORT_ROCM_INFO, YVEX_BACKEND_KIND_ROCM};
    yvex_error err;
    yvex_error_clear(&err);
    if (!argv) {
        yvex_error_set(&err, YVEX_ERR_INVALID_ARG, "rocm-info", "rocm-info arguments are required");
        return command_error(&err, YVEX_ERR_INVALID_ARG);
    }
    if ((argc == 3 && is_help(argv[2])) ||
        (argc == 4 && strcmp(argv[2], "bandwidth") == 0 && is_help(argv[3]))) {
        printf("usage: yvex inspect rocm [bandwidth]\n\n"
               "Reports ROCm facts or runs the bounded bandwidth fixture.\n");
        return 0;
    }
    if (argc == 3 && strcmp(argv[2], "bandwidth") == 0) {
        request.kind = YVEX_BACKEND_REPORT_ROCM_BANDWIDTH;
    } else if (argc != 2) {
        yvex_error_set(&err, YVEX_ERR_INVALID_ARG, "rocm-info",
                       "usage: yvex inspect rocm [bandwidth]");
        return command_error(&err, YVEX_ERR_INVALID_ARG);
    }
    return command_run(&request);
}

/* ---- benchmark sample summary --------------------------------------------------------- */

static int sample_compare(const void *left, const void *right)
{
    const double a = *(const double *)left, b = *(const double *)right;
    return a < b ? -1 : a > b ? 1 : 0;
}

/* seconds to whole nanoseconds, rounding the fraction half up
 * (src/runtime/benchmark.c:388-398) */
static int seconds_ns(double seconds, unsigned long long *output)
{
    double integral_seconds, fractional_seconds;
    unsigned long long integral_ns, fractional_ns;
    if (!isfinite(seconds) || seconds < 0.0) return 0;
    fractional_seconds = modf(seconds, &integral_seconds);
    if (integral_seconds > (double)(ULLONG_MAX / 1000000000ull)) return 0;
    fractional_ns = (unsigned long long)(fractional_seconds * 1000000000.0 + 0.5);
    return yvex_core_u64_mul((unsigned long long)integral_seconds, 1000000000ull, &integral_ns) &&
           yvex_core_u64_add(integral_ns, fractional_ns, output);
}

int yvex_runtime_benchmark_samples_summarize(double *seconds, unsigned long long count,
                                             yvex_runtime_benchmark_timing_distribution *out,
                                             yvex_error *err)
{
    static const struct {
        unsigned int index, percentile;
    } percentiles[] = {{YVEX_RUNTIME_BENCHMARK_P50, 50u},
                       {YVEX_RUNTIME_BENCHMARK_P90, 90u},
                       {YVEX_RUNTIME_BENCHMARK_P95, 95u},
                       {YVEX_RUNTIME_BENCHMARK_P99, 99u}};
    static const char where[] = "runtime.benchmark";
    double values[YVEX_RUNTIME_BENCHMARK_STATISTIC_COUNT];
    double sum = 0.0, squared = 0.0;
    unsigned long long index;
    size_t p;

    if (out) memset(out, 0, sizeof(*out));
    if (!seconds || !out || !count || count > (unsigned long long)(SIZE_MAX / sizeof(*seconds))) {
        yvex_error_set(err, YVEX_ERR_BOUNDS, where,
                       "benchmark samples must be positive, finite, and complete");
        return YVEX_ERR_BOUNDS;
    }
    for (index = 0ull; index < count; ++index) {
        if (!isfinite(seconds[index]) || seconds[index] <= 0.0) {
            yvex_error_set(err, YVEX_ERR_BOUNDS, where,
                           "benchmark samples must be positive, finite, and complete");
            return YVEX_ERR_BOUNDS;
        }
    }
    qsort(seconds, (size_t)count, sizeof(*seconds), sample_compare);
    for (index = 0ull; index < count; ++index) sum += seconds[index];
    values[YVEX_RUNTIME_BENCHMARK_MINIMUM] = seconds[0];
    for (p = 0u; p < sizeof(percentiles) / sizeof(percentiles[0]); ++p)
        values[percentiles[p].index] =
            seconds[(count * percentiles[p].percentile + 99ull) / 100ull - 1ull];
    values[YVEX_RUNTIME_BENCHMARK_MAXIMUM] = seconds[count - 1ull];
    values[YVEX_RUNTIME_BENCHMARK_MEAN] = sum / (double)count;
    for (index = 0ull; index < count; ++index) {
        const double delta = seconds[index] - values[YVEX_RUNTIME_BENCHMARK_MEAN];
        squared += delta * delta;
    }
    values[YVEX_RUNTIME_BENCHMARK_STANDARD_DEVIATION] = sqrt(squared / (double)count);
    for (p = 0u; p < YVEX_RUNTIME_BENCHMARK_STATISTIC_COUNT; ++p) {
        if (!seconds_ns(values[p], &out->values[p])) {
            memset(out, 0, sizeof(*out));
            yvex_error_set(err, YVEX_ERR_BOUNDS, where,
                           "attention benchmark timing is not representable");
            return YVEX_ERR_BOUNDS;
        }
    }
    /* a distribution whose minimum rounds to zero nanoseconds is not evidence
     * (src/runtime/benchmark.c:559-573) */
    if (out->values[YVEX_RUNTIME_BENCHMARK_MINIMUM] == 0ull) {
        memset(out, 0, sizeof(*out));
        yvex_error_set(err, YVEX_ERR_BOUNDS, where,
                       "attention benchmark timing is not representable");
        return YVEX_ERR_BOUNDS;
    }
    out->available = 1;
    yvex_error_clear(err);
    return YVEX_OK;
}

const char *yvex_runtime_benchmark_statistic_name(yvex_runtime_benchmark_statistic statistic)
{
    switch (statistic) {
    case YVEX_RUNTIME_BENCHMARK_MINIMUM: return "minimum_ns";
    case YVEX_RUNTIME_BENCHMARK_P50: return "p50_ns";
    case YVEX_RUNTIME_BENCHMARK_P90: return "p90_ns";
    case YVEX_RUNTIME_BENCHMARK_P95: return "p95_ns";
    case YVEX_RUNTIME_BENCHMARK_P99: return "p99_ns";
    case YVEX_RUNTIME_BENCHMARK_MAXIMUM: return "maximum_ns";
    case YVEX_RUNTIME_BENCHMARK_MEAN: return "mean_ns";
    case YVEX_RUNTIME_BENCHMARK_STANDARD_DEVIATION: return "standard_deviation_ns";
    case YVEX_RUNTIME_BENCHMARK_STATISTIC_COUNT: break;
    }
    return NULL;
}
