// Runs the absorbed BF16 MLA forward and backward once (after one warm call) for rocprofv3, or times them.
// Counterpart of the reference's benchmarks/attention/benchmark_mla.cu: same arguments
// (batch sequence heads kv_rank rope), same constant inputs (benchmark_mla.cu:38-47).  Those inputs
// have a closed form, which is checked here:
//   every score = (C*0.125*0.25 - R*0.0625*0.03125) * scale, so row t attends uniformly over t+1 keys:
//   O = 0.25, LSE[t] = score + ln(t+1);  with dO = 0.015625: dP = delta, dS = 0, so
//   dq_latent = dq_rope = dk_rope = 0 and dLatent[k,:] = H * 0.015625 * (Harm(T) - Harm(k)).
//
//   benchmark_mla [batch=1] [sequence=128] [heads=8] [kv_rank=512] [rope=64] [--timing ...] [--no-check]
#include "mla.h"
#include "profiler_common.h"

int main(int argc, char** argv) {
    using namespace profiler;
    try {
        const int batch = positive_argument(argc, argv, 1, 1, "batch");
        const int sequence = positive_argument(argc, argv, 2, 128, "sequence");
        const int heads = positive_argument(argc, argv, 3, 8, "heads");
        const int rank = positive_argument(argc, argv, 4, 512, "kv_rank");
        const int rope = positive_argument(argc, argv, 5, 64, "rope");
        int first_flag = 1;
        while (first_flag < argc && argv[first_flag][0] != '-') ++first_flag;
        const Options options = parse_options(argc, argv, first_flag);
        const float scale = 1.0F / std::sqrt(static_cast<float>(rank + rope));

        const std::size_t tokens = static_cast<std::size_t>(batch) * sequence;
        const std::size_t query_elements = tokens * heads * rank;
        const std::size_t query_rope_elements = tokens * heads * rope;
        const std::size_t latent_elements = tokens * rank;
        const std::size_t key_rope_elements = tokens * rope;
        const std::size_t rows = tokens * heads;

        DeviceBuffer<__hip_bfloat16> query(query_elements), query_rope(query_rope_elements), latent(latent_elements),
            key_rope(key_rope_elements), output(query_elements), output_gradient(query_elements),
            query_gradient(query_elements), query_rope_gradient(query_rope_elements), latent_gradient(latent_elements),
            key_rope_gradient(key_rope_elements);
        DeviceBuffer<float> logsumexp(rows);
        query.upload(filled(query_elements, 0.125F));
        query_rope.upload(filled(query_rope_elements, -0.0625F));
        latent.upload(filled(latent_elements, 0.25F));
        key_rope.upload(filled(key_rope_elements, 0.03125F));
        output_gradient.upload(filled(query_elements, 0.015625F));

        auto run = [&]() {
            dscuda::mla_compressed_attention_forward_cuda(output.get(), logsumexp.get(), query.get(), query_rope.get(),
                                                          latent.get(), key_rope.get(), batch, sequence, heads, rank,
                                                          rope, scale);
            dscuda::mla_compressed_attention_backward_cuda(
                query_gradient.get(), query_rope_gradient.get(), latent_gradient.get(), key_rope_gradient.get(),
                output_gradient.get(), output.get(), logsumexp.get(), query.get(), query_rope.get(), latent.get(),
                key_rope.get(), batch, sequence, heads, rank, rope, scale);
        };

        run();
        PROFILER_HIP_CHECK(hipDeviceSynchronize());
        std::printf("MLA workload: batch=%d sequence=%d heads=%d kv_rank=%d rope=%d\n", batch, sequence, heads, rank,
                    rope);

        if (options.verify) {
            const double score = (rank * 0.125 * 0.25 - rope * 0.0625 * 0.03125) * static_cast<double>(scale);
            const std::vector<double> harmonic = harmonic_numbers(sequence);
            require("output", worst_error(output.download(), [](std::size_t) { return 0.25; }), 2e-3);
            require("logsumexp", worst_error(logsumexp.download(), [&](std::size_t index) {
                        return score + std::log(static_cast<double>(index % sequence) + 1.0);   // [B,H,T]
                    }), 1e-3);
            require("query_latent gradient", worst_error(query_gradient.download(), [](std::size_t) { return 0.0; }), 1e-3);
            require("query_rope gradient", worst_error(query_rope_gradient.download(), [](std::size_t) { return 0.0; }), 1e-3);
            require("key_rope gradient", worst_error(key_rope_gradient.download(), [](std::size_t) { return 0.0; }), 1e-3);
            // bf16 result of a sum that reaches H * 0.015625 * Harm(T): relative tolerance of one bf16 step
            const double largest = heads * 0.015625 * harmonic[sequence];
            require("kv_latent gradient", worst_error(latent_gradient.download(), [&](std::size_t index) {
                        const int key = static_cast<int>((index / rank) % sequence);   // [B,T,C]
                        return heads * 0.015625 * (harmonic[sequence] - harmonic[key]);
                    }), std::max(2e-3, largest / 128.0));
        }

        if (options.timing.enabled) {
            const TimingResult result = measure_gpu(run, options.timing);
            print_timing("forward+backward", batch, sequence, heads, rank + rope, options.timing, result);
        } else {
            run();   // the launch a profiler looks at: the second of two identical ones
            PROFILER_HIP_CHECK(hipDeviceSynchronize());
        }
        return 0;
    } catch (const std::exception& error) {
        std::fprintf(stderr, "MLA benchmark failed: %s\n", error.what());
        return 1;
    }
}
