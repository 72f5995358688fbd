// Shared host-side pieces of the standalone profiler programs: device buffers,
// event timing, closed-form checks and the timing line the reference's tooling
// parses.  The programs are the counterparts of the reference's
// benchmarks/attention/benchmark_*.cu: one process, one workload, deterministic
// inputs, nothing but the library's own kernels on the GPU -- the shape
// rocprofv3 wants.  Unlike the reference's, each program also checks what the
// kernels returned against the closed form its inputs have, and fails loudly
// if they differ.
#pragma once

#include <hip/hip_bf16.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

namespace profiler {

inline void check(hipError_t status, const char* expression, const char* file, int line) {
    if (status != hipSuccess) {
        throw std::runtime_error(std::string("HIP failure at ") + file + ":" + std::to_string(line) +
                                 " while evaluating " + expression + ": " + hipGetErrorString(status));
    }
}
#define PROFILER_HIP_CHECK(expression) ::profiler::check((expression), #expression, __FILE__, __LINE__)

// Device allocation that frees itself; the library under test never allocates.
template <typename T>
class DeviceBuffer {
public:
    explicit DeviceBuffer(std::size_t elements) : elements_(elements) {
        PROFILER_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&pointer_), std::max<std::size_t>(1, elements) * sizeof(T)));
    }
    DeviceBuffer(const DeviceBuffer&) = delete;
    DeviceBuffer& operator=(const DeviceBuffer&) = delete;
    ~DeviceBuffer() { (void)hipFree(pointer_); }

    T* get() const { return pointer_; }
    std::size_t size() const { return elements_; }

    void upload(const std::vector<T>& host) {
        if (host.size() != elements_) throw std::invalid_argument("upload: size mismatch");
        PROFILER_HIP_CHECK(hipMemcpy(pointer_, host.data(), elements_ * sizeof(T), hipMemcpyHostToDevice));
    }
    std::vector<T> download() const {
        std::vector<T> host(elements_);
        PROFILER_HIP_CHECK(hipMemcpy(host.data(), pointer_, elements_ * sizeof(T), hipMemcpyDeviceToHost));
        return host;
    }

private:
    T* pointer_ = nullptr;
    std::size_t elements_ = 0;
};

inline std::vector<__hip_bfloat16> filled(std::size_t elements, float value) {
    return std::vector<__hip_bfloat16>(elements, __float2bfloat16(value));
}

// Positive integer from the command line (the reference's mains take atoi of
// whatever they are given; a non-positive size is refused here instead).
inline int positive_argument(int argc, char** argv, int index, int fallback, const char* name) {
    if (argc <= index || argv[index][0] == '-') return fallback;
    const int value = std::atoi(argv[index]);
    if (value <= 0) throw std::invalid_argument(std::string(name) + " must be a positive integer");
    return value;
}

struct TimingOptions {   // reference benchmarks/attention/benchmark_flash_attention.cu:19-24
    bool enabled = false;
    int warmup = 10;
    int iterations = 50;
    int trials = 5;
};

struct Options {
    TimingOptions timing;
    bool verify = true;
    bool constant_inputs = false;
    std::string operation = "forward";
    const char* dump_path = nullptr;
};

// Flags after the positional sizes: --timing [--warmup N] [--iterations N] [--trials N], --no-check,
// --constant, --operation NAME; anything else is the path of a raw fp32 dump.
inline Options parse_options(int argc, char** argv, int first) {
    Options options;
    for (int index = first; index < argc; ++index) {
        const char* argument = argv[index];
        auto value_of = [&](const char* flag) {
            if (index + 1 >= argc) throw std::invalid_argument(std::string(flag) + " needs a value");
            const int value = std::atoi(argv[++index]);
            if (value <= 0) throw std::invalid_argument(std::string(flag) + " must be positive");
            return value;
        };
        if (std::strcmp(argument, "--timing") == 0) options.timing.enabled = true;
        else if (std::strcmp(argument, "--warmup") == 0) options.timing.warmup = value_of("--warmup");
        else if (std::strcmp(argument, "--iterations") == 0) options.timing.iterations = value_of("--iterations");
        else if (std::strcmp(argument, "--trials") == 0) options.timing.trials = value_of("--trials");
        else if (std::strcmp(argument, "--no-check") == 0) options.verify = false;
        else if (std::strcmp(argument, "--constant") == 0) options.constant_inputs = true;
        else if (std::strcmp(argument, "--operation") == 0) {
            if (index + 1 >= argc) throw std::invalid_argument("--operation needs a value");
            options.operation = argv[++index];
        } else if (argument[0] == '-' && argument[1] == '-') {
            throw std::invalid_argument(std::string("unknown option ") + argument);
        } else {
            options.dump_path = argument;
        }
    }
    return options;
}

struct TimingResult {
    float median_ms;
    float minimum_ms;
    float maximum_ms;
};

// Warm-up launches, then `trials` event-bracketed groups of `iterations` launches on the null
// stream; per-launch time of each group, median / min / max over the groups
// (the scheme of benchmark_flash_attention.cu:47-83).
template <typename Operation>
TimingResult measure_gpu(Operation operation, const TimingOptions& timing) {
    for (int iteration = 0; iteration < timing.warmup; ++iteration) operation();
    PROFILER_HIP_CHECK(hipDeviceSynchronize());
    hipEvent_t start, stop;
    PROFILER_HIP_CHECK(hipEventCreate(&start));
    PROFILER_HIP_CHECK(hipEventCreate(&stop));
    std::vector<float> measurements(timing.trials);
    for (int trial = 0; trial < timing.trials; ++trial) {
        PROFILER_HIP_CHECK(hipEventRecord(start, nullptr));
        for (int iteration = 0; iteration < timing.iterations; ++iteration) operation();
        PROFILER_HIP_CHECK(hipEventRecord(stop, nullptr));
        PROFILER_HIP_CHECK(hipEventSynchronize(stop));
        PROFILER_HIP_CHECK(hipEventElapsedTime(&measurements[trial], start, stop));
        measurements[trial] /= static_cast<float>(timing.iterations);
    }
    PROFILER_HIP_CHECK(hipEventDestroy(stop));
    PROFILER_HIP_CHECK(hipEventDestroy(start));
    std::sort(measurements.begin(), measurements.end());
    const int trials = timing.trials;
    const float median = trials % 2 == 0 ? 0.5F * (measurements[trials / 2 - 1] + measurements[trials / 2])
                                         : measurements[trials / 2];
    return {median, measurements.front(), measurements.back()};
}

// The line the reference's profile tooling greps for (benchmark_flash_attention.cu:196-214), with the
// same keys; `extra` is appended verbatim (more "key":value pairs, starting with a comma) or empty.
inline void print_timing(const char* operation, int batch, int sequence, int heads, int head_size,
                         const TimingOptions& timing, const TimingResult& result, const std::string& extra = "") {
    std::printf("DSCUDA_TIMING {\"backend\":\"custom\",\"mode\":\"native_eager\",\"operation\":\"%s\",\"batch\":%d,"
                "\"sequence\":%d,\"heads\":%d,\"head_size\":%d,\"warmup\":%d,\"iterations\":%d,\"trials\":%d,"
                "\"median_ms\":%.9g,\"minimum_ms\":%.9g,\"maximum_ms\":%.9g%s}\n",
                operation, batch, sequence, heads, head_size, timing.warmup, timing.iterations, timing.trials,
                result.median_ms, result.minimum_ms, result.maximum_ms, extra.c_str());
}

// Largest |actual - expected(index)| over a bf16 buffer.
template <typename Expected>
double worst_error(const std::vector<__hip_bfloat16>& actual, Expected expected) {
    double worst = 0.0;
    for (std::size_t index = 0; index < actual.size(); ++index) {
        const double value = static_cast<double>(__bfloat162float(actual[index]));
        if (!std::isfinite(value)) return INFINITY;
        worst = std::max(worst, std::fabs(value - expected(index)));
    }
    return worst;
}

template <typename Expected>
double worst_error(const std::vector<float>& actual, Expected expected) {
    double worst = 0.0;
    for (std::size_t index = 0; index < actual.size(); ++index) {
        if (!std::isfinite(actual[index])) return INFINITY;
        worst = std::max(worst, std::fabs(static_cast<double>(actual[index]) - expected(index)));
    }
    return worst;
}

inline void require(const char* what, double error, double tolerance) {
    std::printf("check %-28s max |error| %.3e (tolerance %.1e)\n", what, error, tolerance);
    if (!(error <= tolerance)) {
        throw std::runtime_error(std::string(what) + " differs from its closed form");
    }
}

// Harm(n) = sum_{i=1..n} 1/i for n = 0..count
inline std::vector<double> harmonic_numbers(int count) {
    std::vector<double> harmonic(count + 1, 0.0);
    for (int n = 1; n <= count; ++n) harmonic[n] = harmonic[n - 1] + 1.0 / n;
    return harmonic;
}

// Raw fp32 dump of a bf16 device buffer, for comparison across processes
// (benchmark_flash_attention.cu:31-45).
inline void dump_as_float(const char* path, const std::vector<__hip_bfloat16>& values) {
    std::FILE* file = std::fopen(path, "wb");
    if (file == nullptr) throw std::runtime_error(std::string("cannot open dump file: ") + path);
    std::vector<float> decoded(values.size());
    for (std::size_t index = 0; index < values.size(); ++index) decoded[index] = __bfloat162float(values[index]);
    const std::size_t written = std::fwrite(decoded.data(), sizeof(float), decoded.size(), file);
    std::fclose(file);
    if (written != decoded.size()) throw std::runtime_error(std::string("short write to ") + path);
}

}  // namespace profiler
