// Timing of the simulated K-worker quantized all-reduce on one GPU (the "K = 8 workers x 2048 x 9304, all in one GPU's
// memory" workload) through the aggregator classes. Prints one line per arrangement.
//
//   bench_allreduce [K rows cols nbits steps]        defaults: 8 2048 9304 1 20
//   bench_allreduce K resnet50|speech - nbits steps  a whole gradient set instead of one matrix (ResNet-50's 161
//                                                    parameter matrices; the 429-2048x6-9304 speech network's 16)
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
#include <string>

using namespace cntk_amd;

typedef std::vector<std::pair<size_t, size_t>> Shapes;

static Shapes ResNet50()
{
    Shapes convs = {{147, 64}};
    auto stage = [&](size_t cin, size_t mid, size_t cout, int blocks) {
        convs.insert(convs.end(), {{cin, mid}, {9 * mid, mid}, {mid, cout}, {cin, cout}});
        for (int i = 1; i < blocks; ++i)
            convs.insert(convs.end(), {{cout, mid}, {9 * mid, mid}, {mid, cout}});
    };
    stage(64, 64, 256, 3);
    stage(256, 128, 512, 4);
    stage(512, 256, 1024, 6);
    stage(1024, 512, 2048, 3);
    Shapes all = convs;
    all.push_back({2048, 1000});
    all.push_back({1000, 1});
    for (const auto& c : convs) // batch-normalisation scale and bias per convolution
    {
        all.push_back({c.second, 1});
        all.push_back({c.second, 1});
    }
    return all;
}

static Shapes Speech()
{
    Shapes s = {{429, 2048}};
    for (int i = 0; i < 6; ++i)
        s.push_back({2048, 2048});
    s.push_back({2048, 9304});
    for (int i = 0; i < 7; ++i)
        s.push_back({2048, 1});
    s.push_back({9304, 1});
    return s;
}

int main(int argc, char** argv)
{
    const size_t K = argc > 1 ? std::strtoul(argv[1], nullptr, 10) : 8;
    const std::string what = argc > 2 ? argv[2] : "2048";
    const int nbits = argc > 4 ? std::atoi(argv[4]) : 1;
    const int steps = argc > 5 ? std::atoi(argv[5]) : 20;
    Shapes shapes;
    if (what == "resnet50")
        shapes = ResNet50();
    else if (what == "speech")
        shapes = Speech();
    else if (what == "lstm") // language model: embedding, four LSTM weight matrices, softmax
        shapes = {{100000, 512}, {1024, 4096}, {1024, 4096}, {1024, 4096}, {1024, 4096}, {512, 100000}};
    else
        shapes = {{std::strtoul(what.c_str(), nullptr, 10), argc > 3 ? std::strtoul(argv[3], nullptr, 10) : 9304}};
    try
    {
        // pristine gradients, restored before every step (outside the timed region)
        std::vector<std::vector<std::unique_ptr<Matrix<float>>>> pristine(K), work(K);
        std::mt19937_64 rng(0x1B17 + 4000);
        std::normal_distribution<float> dist(0.0f, 0.01f);
        const double b = nbits;
        double bytes = 0;
        size_t params = 0;
        for (const auto& sh : shapes)
        {
            const double n = (double) sh.first * sh.second, cols = (double) sh.second;
            bytes += K * ((12 + b / 8) * n + 8.0 * cols) + ((8 + (K + 1) * b / 8) * n + (K + 1) * 8.0 * cols) + ((4 + b / 8) * n + 8.0 * cols);
            params += sh.first * sh.second;
        }
        for (size_t r = 0; r < K; ++r)
            for (const auto& sh : shapes)
            {
                std::vector<float> host(sh.first * sh.second);
                for (auto& x : host)
                    x = dist(rng);
                pristine[r].emplace_back(new Matrix<float>(sh.first, sh.second, 0));
                pristine[r].back()->SetValue(host.data());
                work[r].emplace_back(new Matrix<float>(sh.first, sh.second, 0));
            }
        if (shapes.size() == 1)
            std::printf("K=%zu %zux%zu nbits=%d: algorithmic bytes per step %.1f MB\n", K, shapes[0].first, shapes[0].second, nbits, bytes / 1e6);
        else
            std::printf("K=%zu %s (%zu matrices, %zu parameters) nbits=%d: algorithmic bytes per step %.1f MB\n", K, what.c_str(),
                        shapes.size(), params, nbits, bytes / 1e6);

        struct Arrangement { const char* name; bool fused, batched, allWorkers, dedicatedStream; };
        const Arrangement arrangements[] = {
            {"fused stripe reduction, unquantize on worker 0", true, true, false, true},
            {"the same on the main stream (no hand-over event)", true, true, false, false},
            {"fused stripe reduction, unquantize on all workers", true, true, true, true},
            {"reference call sequence (unfused), unquantize on worker 0", false, false, false, true},
        };
        for (const Arrangement& a : arrangements)
        {
            InProcessCluster<float>::Options opt;
            opt.useFusedStripeReduce = a.fused;
            opt.useBatchedCalls = a.batched;
            InProcessCluster<float> cluster(K, 0, nbits, false, true, a.dedicatedStream, opt);
            std::vector<std::vector<Matrix<float>*>> grads(K);
            std::vector<DistGradHeader> headers;
            for (size_t r = 0; r < K; ++r)
            {
                for (auto& m : work[r])
                    grads[r].push_back(m.get());
                headers.emplace_back(1);
            }
            double total = 0, best = 1e30;
            for (int step = -3; step < steps; ++step)
            {
                for (size_t r = 0; r < K; ++r)
                {
                    for (size_t i = 0; i < shapes.size(); ++i)
                        detail::HipCheck(hipMemcpyAsync(work[r][i]->Data(), pristine[r][i]->Data(), work[r][i]->GetNumElements() * sizeof(float),
                                                        hipMemcpyDeviceToDevice, nullptr),
                                         "hipMemcpyAsync");
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
