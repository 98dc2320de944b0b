// Timing of the simulated K-worker quantized all-reduce on one GPU (the "K = 8 workers x 2048 x 9304, all in one GPU's
// memory" workload) through the aggregator classes. Prints one line per arrangement.
//
//   bench_allreduce [K rows cols nbits steps]        defaults: 8 2048 9304 1 20
//
// One step = every worker quantizes its gradient with its residual, every worker reduces its own column stripe over
// all K packed gradients and requantizes it with its stripe residual, the requantized stripes are gathered and the
// packed aggregate is unquantized (on worker 0 only, or on every worker). Time is host wall-clock per step between two
// device synchronisations, i.e. including every launch and wait of the aggregator.
//
// Algorithmic bytes per step (b = nbits, n = rows * cols): K quantizations (12 + b/8) n + 8 cols each, the stripe
// reductions (8 + (K + 1) b/8) n + (K + 1) 8 cols in total, and one unquantization (4 + b/8) n + 8 cols.
#include "../../cntk_amd/cpp/AllReduceDistGradAggregator.h"

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <random>

using namespace cntk_amd;

int main(int argc, char** argv)
{
    const size_t K = argc > 1 ? std::strtoul(argv[1], nullptr, 10) : 8;
    const size_t rows = argc > 2 ? std::strtoul(argv[2], nullptr, 10) : 2048;
    const size_t cols = argc > 3 ? std::strtoul(argv[3], nullptr, 10) : 9304;
    const int nbits = argc > 4 ? std::atoi(argv[4]) : 1;
    const int steps = argc > 5 ? std::atoi(argv[5]) : 20;
    const size_t n = rows * cols;
    try
    {
        // pristine gradients, restored before every step (outside the timed region)
        std::vector<std::unique_ptr<Matrix<float>>> pristine, work;
        std::mt19937_64 rng(0x1B17 + 4000);
        std::normal_distribution<float> dist(0.0f, 0.01f);
        std::vector<float> host(n);
        for (size_t r = 0; r < K; ++r)
        {
            for (auto& x : host)
                x = dist(rng);
            pristine.emplace_back(new Matrix<float>(rows, cols, 0));
            pristine.back()->SetValue(host.data());
            work.emplace_back(new Matrix<float>(rows, cols, 0));
        }
        const double b = nbits;
        const double bytes = K * ((12 + b / 8) * n + 8.0 * cols) + ((8 + (K + 1) * b / 8) * n + (K + 1) * 8.0 * cols) + ((4 + b / 8) * n + 8.0 * cols);
        std::printf("K=%zu %zux%zu nbits=%d: algorithmic bytes per step %.1f MB\n", K, rows, cols, nbits, bytes / 1e6);

        struct Arrangement { const char* name; bool fused, batched, allWorkers; };
        const Arrangement arrangements[] = {
            {"fused stripe reduction, unquantize on worker 0", true, true, false},
            {"fused stripe reduction, unquantize on all workers", true, true, true},
            {"reference call sequence (unfused), unquantize on worker 0", false, false, false},
        };
        for (const Arrangement& a : arrangements)
        {
            InProcessCluster<float>::Options opt;
            opt.useFusedStripeReduce = a.fused;
            opt.useBatchedCalls = a.batched;
            InProcessCluster<float> cluster(K, 0, nbits, false, true, true, opt);
            std::vector<std::vector<Matrix<float>*>> grads(K);
            std::vector<DistGradHeader> headers;
            for (size_t r = 0; r < K; ++r)
            {
                grads[r].push_back(work[r].get());
                headers.emplace_back(1);
            }
            double total = 0, best = 1e30;
            for (int step = -3; step < steps; ++step)
            {
                for (size_t r = 0; r < K; ++r)
                {
                    detail::HipCheck(hipMemcpy(work[r]->Data(), pristine[r]->Data(), n * sizeof(float), hipMemcpyDeviceToDevice), "hipMemcpy");
                    headers[r].Clear();
                    headers[r].numSamples = 256;
                }
                detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
                const auto t0 = std::chrono::steady_clock::now();
                cluster.AggregateGradients(grads, headers, step == -3, a.allWorkers);
                detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
                const double us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
                if (step >= 0)
                {
                    total += us;
                    best = std::min(best, us);
                }
            }
            const double avg = total / steps;
            std::printf("%-62s avg %9.1f us  best %9.1f us  %7.1f GB/s algorithmic (%4.1f%% of 8 TB/s)\n", a.name, avg, best, bytes / avg / 1e3,
                        bytes / avg / 1e3 / 80.0);
            std::fflush(stdout);
        }
    }
    catch (const std::exception& e)
    {
        std::fprintf(stderr, "bench_allreduce: %s\n", e.what());
        return 1;
    }
    return 0;
}
