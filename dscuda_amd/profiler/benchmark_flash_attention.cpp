// Runs one BF16 causal flash-attention forward for rocprofv3, times it, or dumps its output.
// Counterpart of the reference's benchmarks/attention/benchmark_flash_attention.cu: same arguments
// (batch sequence heads head_size operation [--timing --warmup N --iterations N --trials N] [dump path]),
// the same index-pattern inputs (benchmark_flash_attention.cu:126-136, shared with the comparison script
// reference/python/flash_attention_official.py:39-48) so that dumps of the two implementations can be
// compared across processes, the same DSCUDA_TIMING line.  Checked here: the first row of every head
// sees one key, so O[0] = V[0] and LSE[0] = scale * q0.k0.
//
//   benchmark_flash_attention [batch=2] [sequence=256] [heads=8] [head_size=128] [forward] [flags] [dump.f32]
#include "flash_attention.h"
#include "profiler_common.h"

int main(int argc, char** argv) {
    using namespace profiler;
    try {
        const int batch = positive_argument(argc, argv, 1, 2, "batch");
        const int sequence = positive_argument(argc, argv, 2, 256, "sequence");
        const int heads = positive_argument(argc, argv, 3, 8, "heads");
        const int head_size = positive_argument(argc, argv, 4, 128, "head_size");
        int first_flag = 5;
        std::string operation = "forward";
        if (argc > 5 && argv[5][0] != '-') {
            operation = argv[5];
            first_flag = 6;
        }
        first_flag = std::min(first_flag, argc);
        const Options options = parse_options(argc, argv, first_flag);
        if (operation != "forward") throw std::runtime_error("only forward is supported");

        const float scale = 1.0F / std::sqrt(static_cast<float>(head_size));
        const std::size_t activations = static_cast<std::size_t>(batch) * sequence * heads * head_size;
        const std::size_t rows = static_cast<std::size_t>(batch) * heads * sequence;

        std::vector<__hip_bfloat16> host_query(activations), host_key(activations), host_value(activations);
        for (std::size_t index = 0; index < activations; ++index) {
            host_query[index] = __float2bfloat16(static_cast<float>(static_cast<int>((index * 17) % 101) - 50) / 64.0F);
            host_key[index] = __float2bfloat16(static_cast<float>(static_cast<int>((index * 23) % 97) - 48) / 61.0F);
            host_value[index] = __float2bfloat16(static_cast<float>(static_cast<int>((index * 31) % 89) - 44) / 59.0F);
        }
        DeviceBuffer<__hip_bfloat16> query(activations), key(activations), value(activations), output(activations);
        DeviceBuffer<float> logsumexp(rows);
        query.upload(host_query);
        key.upload(host_key);
        value.upload(host_value);

        auto forward = [&]() {
            dscuda::flash_attention_forward_cuda(output.get(), logsumexp.get(), query.get(), key.get(), value.get(),
                                                 batch, sequence, heads, heads, head_size, scale);
        };
        std::printf("FlashAttention workload: B=%d T=%d H=%d D=%d operation=%s\n", batch, sequence, heads, head_size,
                    operation.c_str());

        forward();
        PROFILER_HIP_CHECK(hipDeviceSynchronize());
        if (options.verify) {
            const std::vector<__hip_bfloat16> host_output = output.download();
            const std::vector<float> host_lse = logsumexp.download();
            double output_error = 0.0, lse_error = 0.0;
            for (int b = 0; b < batch; ++b) {
                for (int h = 0; h < heads; ++h) {
                    const std::size_t row = (static_cast<std::size_t>(b) * sequence * heads + h) * head_size;   // token 0
                    double dot = 0.0;
                    for (int d = 0; d < head_size; ++d) {
                        dot += static_cast<double>(__bfloat162float(host_query[row + d])) * __bfloat162float(host_key[row + d]);
                        output_error = std::max(output_error, std::fabs(static_cast<double>(__bfloat162float(host_output[row + d])) -
                                                                       __bfloat162float(host_value[row + d])));
                    }
                    const float lse = host_lse[(static_cast<std::size_t>(b) * heads + h) * sequence];
                    lse_error = std::max(lse_error, std::fabs(lse - dot * scale));
                }
            }
            require("first-row output", output_error, 4e-3);
            require("first-row logsumexp", lse_error, 1e-3);
        }

        if (options.timing.enabled) {
            const TimingResult result = measure_gpu(forward, options.timing);
            print_timing(operation.c_str(), batch, sequence, heads, head_size, options.timing, result);
        } else {
            forward();
            PROFILER_HIP_CHECK(hipDeviceSynchronize());
        }
        if (options.dump_path != nullptr) {
            forward();
            PROFILER_HIP_CHECK(hipDeviceSynchronize());
            dump_as_float(options.dump_path, output.download());
        }
        return 0;
    } catch (const std::exception& error) {
        std::fprintf(stderr, "FlashAttention benchmark failed: %s\n", error.what());
        return 1;
    }
}
