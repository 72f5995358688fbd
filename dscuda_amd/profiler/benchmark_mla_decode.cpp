// Runs the absorbed split-KV decode once (after one warm call) for rocprofv3, or times it.
// Counterpart of the reference's benchmarks/attention/benchmark_mla_decode.cu: same arguments
// (batch context heads kv_rank rope splits), 64-token pages, identity block table, every sequence
// `context` long, the same constant inputs (benchmark_mla_decode.cu:42-48).  Closed form, checked here:
//   every score = (C+R) * 0.125 * 0.25 * scale, so O = 0.25 and LSE = score + ln(context).
//
//   benchmark_mla_decode [batch=2] [context=1024] [heads=16] [kv_rank=512] [rope=64] [splits=8]
//                        [--timing ...] [--no-check]
#include "mla.h"
#include "profiler_common.h"

#include <numeric>

int main(int argc, char** argv) {
    using namespace profiler;
    try {
        const int batch = positive_argument(argc, argv, 1, 2, "batch");
        const int context = positive_argument(argc, argv, 2, 1024, "context");
        const int heads = positive_argument(argc, argv, 3, 16, "heads");
        const int rank = positive_argument(argc, argv, 4, 512, "kv_rank");
        const int rope = positive_argument(argc, argv, 5, 64, "rope");
        const int splits = positive_argument(argc, argv, 6, 8, "splits");
        int first_flag = 1;
        while (first_flag < argc && argv[first_flag][0] != '-') ++first_flag;
        const Options options = parse_options(argc, argv, first_flag);

        constexpr int page_size = 64;
        const int pages = (context + page_size - 1) / page_size;
        const int width = rank + rope;
        const float scale = 1.0F / std::sqrt(static_cast<float>(width));
        const std::size_t query_elements = static_cast<std::size_t>(batch) * heads * width;
        const std::size_t cache_elements = static_cast<std::size_t>(batch) * pages * page_size * width;
        const std::size_t output_elements = static_cast<std::size_t>(batch) * heads * rank;
        const std::size_t rows = static_cast<std::size_t>(batch) * heads;
        const std::size_t workspace_elements = dscuda::mla_decode_workspace_elements(batch, heads, splits, rank);

        DeviceBuffer<__hip_bfloat16> query(query_elements), cache(cache_elements), output(output_elements);
        DeviceBuffer<int> block_table(static_cast<std::size_t>(batch) * pages), lengths(batch);
        DeviceBuffer<float> logsumexp(rows), workspace(workspace_elements);
        query.upload(filled(query_elements, 0.125F));
        cache.upload(filled(cache_elements, 0.25F));
        std::vector<int> table(static_cast<std::size_t>(batch) * pages);
        std::iota(table.begin(), table.end(), 0);
        block_table.upload(table);
        lengths.upload(std::vector<int>(batch, context));

        auto run = [&]() {
            dscuda::mla_decode_forward_cuda(output.get(), logsumexp.get(), query.get(), cache.get(), block_table.get(),
                                            lengths.get(), workspace.get(), batch, heads, rank, rope, page_size, pages,
                                            splits, scale);
        };

        run();
        PROFILER_HIP_CHECK(hipDeviceSynchronize());
        std::printf("MLA decode workload: batch=%d context=%d heads=%d kv_rank=%d rope=%d page=%d splits=%d\n", batch,
                    context, heads, rank, rope, page_size, splits);

        if (options.verify) {
            const double score = width * 0.125 * 0.25 * static_cast<double>(scale);
            require("output", worst_error(output.download(), [](std::size_t) { return 0.25; }), 2e-3);
            require("logsumexp", worst_error(logsumexp.download(), [&](std::size_t) {
                        return score + std::log(static_cast<double>(context));
                    }), 1e-3);
        }

        if (options.timing.enabled) {
            const TimingResult result = measure_gpu(run, options.timing);
            const double bytes = static_cast<double>(batch) * context * width * 2.0 + query_elements * 2.0 +
                                 output_elements * 2.0 + rows * 4.0;
            char extra[160];
            std::snprintf(extra, sizeof(extra), ",\"splits\":%d,\"algorithmic_bytes\":%.0f,\"gb_per_s\":%.6g", splits,
                          bytes, bytes / (result.median_ms * 1e6));
            print_timing("decode", batch, context, heads, width, options.timing, result, extra);
        } else {
            run();
            PROFILER_HIP_CHECK(hipDeviceSynchronize());
        }
        return 0;
    } catch (const std::exception& error) {
        std::fprintf(stderr, "MLA decode benchmark failed: %s\n", error.what());
        return 1;
    }
}
