// hgemm: benchmark / check driver for the gfx950 HGEMM library.  Counterpart of the
// reference's main (src/main.cu:47-131): parse flags, print the device banner, build the
// Tester, evaluate the vendor library first (it becomes the 100 % line), then every
// hand-written variant of the default run.
#include <omp.h>

#include <string>

#include "flags.h"
#include "tester.h"

using namespace hgemm;

static void write_json(const std::string &path, const Tester &tester, size_t M, size_t N, size_t K, uint64_t seed,
                       const hipDeviceProp_t &prop) {
    FILE *f = fopen(path.c_str(), "w");
    HGEMM_CHECK_MSG(f != nullptr, "cannot write %s", path.c_str());
    fprintf(f, "{\"device\": \"%s\", \"compute_units\": %d, \"clock_mhz\": %.0f, \"M\": %zu, \"N\": %zu, \"K\": %zu,\n",
            prop.name, prop.multiProcessorCount, prop.clockRate * 1e-3, M, N, K);
    fprintf(f, " \"seed\": %llu, \"a_checksum\": \"0x%016llx\", \"b_checksum\": \"0x%016llx\",\n",
            (unsigned long long)seed, (unsigned long long)tester.checksumA(), (unsigned long long)tester.checksumB());
    fprintf(f, " \"flops\": %.6e, \"bytes\": %.6e, \"results\": [\n", 2.0 * M * N * K, hgemm_bytes(M, N, K));
    const auto &recs = tester.records();
    for (size_t i = 0; i < recs.size(); ++i) {
        const EvalRecord &r = recs[i];
        fprintf(f,
                "  {\"name\": \"%s\", \"ms\": %.6f, \"tflops\": %.3f, \"gbps\": %.1f, \"shader_mhz\": %.0f, \"pct_of_first\": %.2f, "
                "\"checked\": %s, \"pass\": %s, \"max_diff\": %.6g, \"avg_diff\": %.6g, \"rel_err\": %.6g}%s\n",
                r.name.c_str(), r.ms, r.tflops, r.gbps, r.shader_mhz, r.pct_of_base, r.checked ? "true" : "false",
                r.pass ? "true" : "false", r.max_diff, r.avg_diff, r.rel_err, i + 1 < recs.size() ? "," : "");
    }
    fprintf(f, " ]}\n");
    fclose(f);
}

int main(int argc, char *argv[]) {
    Flags flags;
    flags.define("M", "512", "M");
    flags.define("N", "2048", "N");
    flags.define("K", "1024", "K");
    flags.define("enable_mfma", "true", "evaluate the tiled MFMA variants");
    flags.define("enable_naive", "false", "also evaluate the naive / base variants left out of the default run");
    flags.define("enable_vendor", "true", "evaluate hipBLASLt first (the 100% line)");
    flags.define("variant", "", "evaluate only this variant (display or symbol name)");
    flags.define("warmup_iterations", "1", "warmup iteration numbers and average the result");
    flags.define("profiling_iterations", "10", "profiling iteration numbers and average the result");
    flags.define("sleep_duration", "100", "sleep_milliseconds between profiling");
    flags.define("enable_check", "false", "check the GPU result against the hipBLASLt result");
    flags.define("cpu_procs", std::to_string(omp_get_num_procs()), "processor num used of CPU");
    flags.define("gpu_rank", "0", "the used GPU rank");
    flags.define("seed", "20230212", "seed of the input matrices");
    flags.define("dist_a", "uniform", "distribution of A: uniform[:lo:hi] | normal[:sigma | :mean:sigma] | zero");
    flags.define("dist_b", "uniform", "distribution of B");
    flags.define("rotate_mb", "0", "cycle over operand sets totalling at least this many MB (HBM-cold timing)");
    flags.define("json", "", "also write the results to this file as JSON");
    flags.define("fill_only", "false", "generate A and B on the host, print their checksums and exit (no GPU needed)");
    flags.parse(argc, argv);

    const size_t M = flags.u64("M"), N = flags.u64("N"), K = flags.u64("K");
    const int cpu_procs = (int)flags.u64("cpu_procs");
    const int gpu_rank = (int)flags.u64("gpu_rank");
    HGEMM_CHECK_GT(cpu_procs, 0);

    omp_set_num_threads(cpu_procs);
    if (flags.boolean("fill_only")) {
        std::vector<_Float16> a(M * K), b(K * N);
        fill_host(a.data(), a.size(), flags.u64("seed"), 1, parse_fill(flags.str("dist_a")));
        fill_host(b.data(), b.size(), flags.u64("seed"), 2, parse_fill(flags.str("dist_b")));
        printf("{\"M\": %zu, \"N\": %zu, \"K\": %zu, \"seed\": %zu, \"a_checksum\": \"0x%016llx\", \"b_checksum\": \"0x%016llx\"}\n",
               M, N, K, flags.u64("seed"), (unsigned long long)checksum64(a.data(), a.size()),
               (unsigned long long)checksum64(b.data(), b.size()));
        return 0;
    }
    HGEMM_CHECK_HIP_ERROR(hipSetDevice(gpu_rank));

    hipDeviceProp_t prop;
    HGEMM_CHECK_HIP_ERROR(hipGetDeviceProperties(&prop, gpu_rank));
    HLOG("HIP HGEMM start with %d CPU processes on the %d-th GPU: %s (%s)", cpu_procs, gpu_rank, prop.name,
         prop.gcnArchName);
    int driver_version = 0, runtime_version = 0;
    HGEMM_CHECK_HIP_ERROR(hipDriverGetVersion(&driver_version));
    HGEMM_CHECK_HIP_ERROR(hipRuntimeGetVersion(&runtime_version));
    HLOG("HIP driver version / runtime version: %d / %d, library: %s", driver_version, runtime_version,
         hgemm_version());
    HLOG("%d compute units, 4 SIMDs/CU, wavefront size: %d", prop.multiProcessorCount, prop.warpSize);
    HLOG("GPU max clock rate: %.0f MHz (%0.2f GHz)", prop.clockRate * 1e-3, prop.clockRate * 1e-6);
    HLOG("Memory clock rate: %.0f MHz (%0.2f GHz)", prop.memoryClockRate * 1e-3, prop.memoryClockRate * 1e-6);
    HLOG("Memory bus width: %d-bit", prop.memoryBusWidth);
    HLOG("Total amount of global memory: %.0f MBytes (%zu Bytes)", (double)prop.totalGlobalMem / 1048576,
         prop.totalGlobalMem);
    HLOG("Total amount of LDS per block: %.0f KBytes (%zu Bytes)", (double)prop.sharedMemPerBlock / 1024,
         prop.sharedMemPerBlock);
    HLOG("Total LDS per compute unit: %.0f KBytes (%zu Bytes)", (double)prop.maxSharedMemoryPerMultiProcessor / 1024,
         prop.maxSharedMemoryPerMultiProcessor);
    HLOG("L2 cache size: %.0f KBytes (%d Bytes)", (double)prop.l2CacheSize / 1024, prop.l2CacheSize);
    HLOG("Total number of registers available per block: %d", prop.regsPerBlock);
    HLOG("Max number of threads per compute unit: %d", prop.maxThreadsPerMultiProcessor);
    HLOG("Max number of threads per block: %d", prop.maxThreadsPerBlock);
    HLOG("Dense FP16 MFMA peak used for percentages: 2500 TFLOPS; HBM peak: 8000 GB/s");

    HLOG("A (%zu x %zu) * B (%zu x %zu) = C (%zu x %zu)", M, K, K, N, M, N);
    HLOG(
        "Profiling: enable mfma: %d, enable naive: %d, warmup iterations: %zu, profiling iterations: %zu, sleep "
        "duration: %zu ms, enable check: %d, seed: %zu, A ~ %s, B ~ %s",
        (int)flags.boolean("enable_mfma"), (int)flags.boolean("enable_naive"), flags.u64("warmup_iterations"),
        flags.u64("profiling_iterations"), flags.u64("sleep_duration"), (int)flags.boolean("enable_check"),
        flags.u64("seed"), flags.str("dist_a").c_str(), flags.str("dist_b").c_str());

    Tester tester(M, N, K, flags.u64("warmup_iterations"), flags.u64("profiling_iterations"),
                  flags.u64("sleep_duration"), flags.boolean("enable_check"), flags.u64("seed"),
                  parse_fill(flags.str("dist_a")), parse_fill(flags.str("dist_b")), flags.u64("rotate_mb"));

    if (flags.boolean("enable_vendor")) tester.evaluate(hgemm_hipblaslt, "Hipblaslt-Gemm");

    const std::string only = flags.str("variant");
    if (!only.empty()) {
        const int idx = hgemm_variant_find(only.c_str());
        HGEMM_CHECK_MSG(idx >= 0, "unknown variant '%s'", only.c_str());
        HGEMM_CHECK_MSG(hgemm_variant_supports(idx, M, N, K), "%s cannot run M=%zu N=%zu K=%zu", only.c_str(), M, N, K);
        tester.evaluate(hgemm_variant_fn(idx), hgemm_variant_name(idx));
    } else if (flags.boolean("enable_mfma")) {
        for (int i = 0; i < hgemm_variant_count(); ++i) {
            if (!hgemm_variant_in_default_run(i) && !flags.boolean("enable_naive")) continue;
            if (!hgemm_variant_supports(i, M, N, K)) {
                HLOG("Skipping %s: shape not supported by this variant", hgemm_variant_name(i));
                continue;
            }
            tester.evaluate(hgemm_variant_fn(i), hgemm_variant_name(i));
        }
    }

    if (!flags.str("json").empty()) write_json(flags.str("json"), tester, M, N, K, flags.u64("seed"), prop);

    if (tester.failures() > 0) {
        HLOG("Done with %zu failed check(s)", tester.failures());
        return EXIT_FAILURE;
    }
    HLOG("Done");
    return 0;
}
