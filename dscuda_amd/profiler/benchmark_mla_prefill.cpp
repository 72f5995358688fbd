// Runs the per-head MLA prefill forward (and backward) for rocprofv3, or times them: the workloads of the
// headline metric (d_qk = 192 = 128 nope + 64 rope, d_v = 128), which the reference has no kernel for.
// Inputs are index patterns in (-1, 1) (the construction of benchmark_flash_attention.cu:126-136 with other
// constants), or constants with --constant.  Checked here:
//   always: the first row of every head sees one key: O[0] = V[0], LSE[0] = scale * q0.k0;
//   --constant (q = 0.125, k = 0.25, v = 0.5, dO = 0.015625): O = 0.5, LSE[t] = d_qk/32 * scale + ln(t+1),
//   dS = 0 so dQ = dK = 0, dV[k,:] = 0.015625 * (Harm(S) - Harm(k)).
//
//   benchmark_mla_prefill [batch=1] [sequence=4096] [heads=128] [d_qk=192] [d_v=128]
//                         [--operation forward|backward|both] [--constant] [--timing ...] [--no-check]
#include "mla.h"
#include "profiler_common.h"

int main(int argc, char** argv) {
    using namespace profiler;
    try {
        const int batch = positive_argument(argc, argv, 1, 1, "batch");
        const int sequence = positive_argument(argc, argv, 2, 4096, "sequence");
        const int heads = positive_argument(argc, argv, 3, 128, "heads");
        const int d_qk = positive_argument(argc, argv, 4, 192, "d_qk");
        const int d_v = positive_argument(argc, argv, 5, 128, "d_v");
        int first_flag = 1;
        while (first_flag < argc && argv[first_flag][0] != '-') ++first_flag;
        const Options options = parse_options(argc, argv, first_flag);
        const bool with_forward = options.operation == "forward" || options.operation == "both";
        const bool with_backward = options.operation == "backward" || options.operation == "both";
        if (!with_forward && !with_backward) throw std::invalid_argument("--operation is forward, backward or both");

        const float scale = 1.0F / std::sqrt(static_cast<float>(d_qk));
        const std::size_t tokens = static_cast<std::size_t>(batch) * sequence;
        const std::size_t qk_elements = tokens * heads * d_qk;
        const std::size_t v_elements = tokens * heads * d_v;
        const std::size_t rows = tokens * heads;

        std::vector<__hip_bfloat16> host_query(qk_elements), host_key(qk_elements), host_value(v_elements),
            host_gradient(v_elements);
        if (options.constant_inputs) {
            host_query = filled(qk_elements, 0.125F);
            host_key = filled(qk_elements, 0.25F);
            host_value = filled(v_elements, 0.5F);
            host_gradient = filled(v_elements, 0.015625F);
        } else {
            for (std::size_t index = 0; index < qk_elements; ++index) {
                host_query[index] = __float2bfloat16(static_cast<float>(static_cast<int>((index * 19) % 103) - 51) / 104.0F);
                host_key[index] = __float2bfloat16(static_cast<float>(static_cast<int>((index * 29) % 107) - 53) / 108.0F);
            }
            for (std::size_t index = 0; index < v_elements; ++index) {
                host_value[index] = __float2bfloat16(static_cast<float>(static_cast<int>((index * 37) % 109) - 54) / 110.0F);
                host_gradient[index] = __float2bfloat16(static_cast<float>(static_cast<int>((index * 41) % 113) - 56) / 57.0F);
            }
        }

        DeviceBuffer<__hip_bfloat16> query(qk_elements), key(qk_elements), value(v_elements), output(v_elements);
        DeviceBuffer<float> logsumexp(rows);
        query.upload(host_query);
        key.upload(host_key);
        value.upload(host_value);

        auto forward = [&]() {
            dscuda::mla_prefill_forward_cuda(output.get(), logsumexp.get(), query.get(), key.get(), value.get(), batch,
                                             sequence, heads, d_qk, d_v, scale);
        };
        std::printf("MLA prefill workload: batch=%d sequence=%d heads=%d d_qk=%d d_v=%d operation=%s inputs=%s\n", batch,
                    sequence, heads, d_qk, d_v, options.operation.c_str(), options.constant_inputs ? "constant" : "pattern");

        forward();   // the backward needs its results whatever is profiled
        PROFILER_HIP_CHECK(hipDeviceSynchronize());
        if (options.verify) {
            const std::vector<__hip_bfloat16> host_output = output.download();
            const std::vector<float> host_lse = logsumexp.download();
            double output_error = 0.0, lse_error = 0.0;
            for (int b = 0; b < batch; ++b) {
                for (int h = 0; h < heads; ++h) {
                    const std::size_t token0 = static_cast<std::size_t>(b) * sequence * heads + h;
                    double dot = 0.0;
                    for (int d = 0; d < d_qk; ++d) {
                        dot += static_cast<double>(__bfloat162float(host_query[token0 * d_qk + d])) *
                               __bfloat162float(host_key[token0 * d_qk + d]);
                    }
                    for (int d = 0; d < d_v; ++d) {
                        output_error = std::max(output_error,
                                                std::fabs(static_cast<double>(__bfloat162float(host_output[token0 * d_v + d])) -
                                                          __bfloat162float(host_value[token0 * d_v + d])));
                    }
                    const float lse = host_lse[(static_cast<std::size_t>(b) * heads + h) * sequence];
                    lse_error = std::max(lse_error, std::fabs(lse - dot * scale));
                }
            }
            require("first-row output", output_error, 4e-3);
            require("first-row logsumexp", lse_error, 1e-3);
            if (options.constant_inputs) {
                const double score = d_qk * 0.125 * 0.25 * static_cast<double>(scale);
                require("output", worst_error(host_output, [](std::size_t) { return 0.5; }), 4e-3);
                require("logsumexp", worst_error(host_lse, [&](std::size_t index) {
                            return score + std::log(static_cast<double>(index % sequence) + 1.0);
                        }), 1e-3);
            }
        }

        if (!with_backward) {
            if (options.timing.enabled) {
                const TimingResult result = measure_gpu(forward, options.timing);
                const double flops = static_cast<double>(batch) * heads * (0.5 * sequence * sequence) * 2.0 * (d_qk + d_v);
                char extra[128];
                std::snprintf(extra, sizeof(extra), ",\"head_size_v\":%d,\"algorithmic_flops\":%.0f,\"tflops\":%.6g", d_v, flops,
                              flops / (result.median_ms * 1e9));
                print_timing("forward", batch, sequence, heads, d_qk, options.timing, result, extra);
            } else {
                forward();
                PROFILER_HIP_CHECK(hipDeviceSynchronize());
            }
            return 0;
        }

        DeviceBuffer<__hip_bfloat16> output_gradient(v_elements), query_gradient(qk_elements), key_gradient(qk_elements),
            value_gradient(v_elements);
        DeviceBuffer<float> workspace(dscuda::mla_prefill_backward_workspace_elements(batch, sequence, heads, d_qk, d_v));
        output_gradient.upload(host_gradient);
        auto backward = [&]() {
            dscuda::mla_prefill_backward_cuda(query_gradient.get(), key_gradient.get(), value_gradient.get(),
                                              output_gradient.get(), output.get(), logsumexp.get(), query.get(), key.get(),
                                              value.get(), workspace.get(), batch, sequence, heads, d_qk, d_v, scale);
        };
        auto profiled = [&]() {
            if (with_forward) forward();
            backward();
        };
        backward();
        PROFILER_HIP_CHECK(hipDeviceSynchronize());
        if (options.verify && options.constant_inputs) {
            const std::vector<double> harmonic = harmonic_numbers(sequence);
            require("query gradient", worst_error(query_gradient.download(), [](std::size_t) { return 0.0; }), 1e-3);
            require("key gradient", worst_error(key_gradient.download(), [](std::size_t) { return 0.0; }), 1e-3);
            const double largest = 0.015625 * harmonic[sequence];
            require("value gradient", worst_error(value_gradient.download(), [&](std::size_t index) {
                        const int key_index = static_cast<int>((index / (static_cast<std::size_t>(heads) * d_v)) % sequence);
                        return 0.015625 * (harmonic[sequence] - harmonic[key_index]);   // [B,S,H,d_v]
                    }), std::max(1e-3, largest / 128.0));
        }
        if (options.timing.enabled) {
            const TimingResult result = measure_gpu(profiled, options.timing);
            const double pairs = static_cast<double>(batch) * heads * (0.5 * sequence * sequence);
            const double flops = pairs * 2.0 * (3.0 * d_qk + 2.0 * d_v) + (with_forward ? pairs * 2.0 * (d_qk + d_v) : 0.0);
            char extra[128];
            std::snprintf(extra, sizeof(extra), ",\"head_size_v\":%d,\"algorithmic_flops\":%.0f,\"tflops\":%.6g", d_v, flops,
                          flops / (result.median_ms * 1e9));
            print_timing(with_forward ? "forward+backward" : "backward", batch, sequence, heads, d_qk, options.timing, result,
                         extra);
        } else {
            profiled();
            PROFILER_HIP_CHECK(hipDeviceSynchronize());
        }
        return 0;
    } catch (const std::exception& error) {
        std::fprintf(stderr, "MLA prefill benchmark failed: %s\n", error.what());
        return 1;
    }
}
