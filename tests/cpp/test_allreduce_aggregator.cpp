// Tests of the quantized all-reduce aggregator (cntk_amd/cpp/AllReduceDistGradAggregator.h) with K workers in one
// process on one GPU. The checker is the CPU oracle's restatement of the same dataflow (oracle_allreduce).
//
//   * every worker ends with the same aggregated gradients (what the reference's distributed tests assert:
//     bindings/python/cntk/learners/tests/distributed_learner_test.py:101-128);
//   * the fused stripe reduction, the batched calls and the dedicated stream change nothing: bit-identical gradients,
//     residuals and stripe residuals against the reference's sequence of per-matrix calls on the main stream;
//   * 32 bits: the aggregate equals the plain fp32 sum in the documented order (the reference's own known answer,
//     Tests/EndToEndTests/CNTKv2Library/EndToEndTests/FrameMode.cpp:112-116);
//   * 1, 2, 4 bits over several carried steps: aggregated gradients against the oracle within 1e-4 of the value range
//     with at most 0.1 % outliers (the reference unit test's GPU tolerance), residuals carried on both sides;
//   * headers are summed; a worker without samples contributes zeros; resetState clears all residuals.
#include "../../cntk_amd/cpp/AllReduceDistGradAggregator.h"
#include "../../oracle/quantizer_oracle.h"

#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>

using namespace cntk_amd;

static int g_failures = 0;
#define CHECK(cond, ...)                                                                                               \
    do                                                                                                                 \
    {                                                                                                                  \
        if (!(cond))                                                                                                   \
        {                                                                                                              \
            if (g_failures < 20)                                                                                       \
            {                                                                                                          \
                std::fprintf(stderr, "CHECK failed %s:%d: %s  ", __FILE__, __LINE__, #cond);                         \
                std::fprintf(stderr, __VA_ARGS__);                                                                     \
                std::fprintf(stderr, "\n");                                                                            \
            }                                                                                                          \
            g_failures++;                                                                                              \
        }                                                                                                              \
    } while (0)

typedef std::vector<std::pair<size_t, size_t>> Shapes;

static std::vector<float> Gaussian(size_t n, float sigma, unsigned long seed)
{
    std::mt19937_64 rng(seed);
    std::normal_distribution<float> d(0.0f, sigma);
    std::vector<float> a(n);
    for (auto& x : a)
        x = d(rng);
    return a;
}

struct WorkerSet
{
    std::vector<std::unique_ptr<Matrix<float>>> owned;
    std::vector<Matrix<float>*> ptrs;
};

static std::vector<WorkerSet> MakeGradients(const Shapes& shapes, size_t K, const std::vector<std::vector<std::vector<float>>>& host)
{
    std::vector<WorkerSet> sets(K);
    for (size_t r = 0; r < K; ++r)
        for (size_t i = 0; i < shapes.size(); ++i)
        {
            sets[r].owned.emplace_back(new Matrix<float>(shapes[i].first, shapes[i].second, 0));
            sets[r].owned.back()->SetValue(host[r][i].data());
            sets[r].ptrs.push_back(sets[r].owned.back().get());
        }
    return sets;
}

static bool SameBits(const Matrix<float>& a, const Matrix<float>& b)
{
    if (a.GetNumElements() != b.GetNumElements())
        return false;
    auto x = a.CopyToArray(), y = b.CopyToArray();
    return std::memcmp(x.get(), y.get(), a.GetNumElements() * sizeof(float)) == 0;
}

// Runs `steps` aggregations with the given options; returns the clusters' final state for comparison.
struct RunResult
{
    std::vector<std::vector<std::vector<float>>> gradients; // [step][matrix] of worker 0
    std::unique_ptr<InProcessCluster<float>> cluster;
    std::vector<WorkerSet> last;
};

static RunResult Run(const Shapes& shapes, size_t K, int nBits, bool zeroThr, bool selfStripeQuantized, bool useAsync, bool fused, bool batched,
                     int steps, unsigned long seed, bool checkAllWorkersEqual, bool clusterBatching = true)
{
    RunResult out;
    InProcessCluster<float>::Options opt;
    opt.useFusedStripeReduce = fused;
    opt.useBatchedCalls = batched;
    opt.useClusterBatching = clusterBatching;
    out.cluster.reset(new InProcessCluster<float>(K, 0, nBits, zeroThr, selfStripeQuantized, useAsync, opt));
    for (int step = 0; step < steps; ++step)
    {
        std::vector<std::vector<std::vector<float>>> host(K);
        for (size_t r = 0; r < K; ++r)
            for (size_t i = 0; i < shapes.size(); ++i)
                host[r].push_back(Gaussian(shapes[i].first * shapes[i].second, 0.01f, seed + 1000 * step + 10 * r + i));
        std::vector<WorkerSet> sets = MakeGradients(shapes, K, host);
        std::vector<std::vector<Matrix<float>*>> grads;
        std::vector<DistGradHeader> headers;
        for (size_t r = 0; r < K; ++r)
        {
            grads.push_back(sets[r].ptrs);
            headers.emplace_back(2);
            headers.back().numSamples = 10 + r;
            headers.back().numSamplesWithLabel = 9 + r;
            headers.back().criterion = 1.5 * (double) (r + 1);
            headers.back().evalErrors[0] = {0.25 * (double) r, 10 + r};
            headers.back().evalErrors[1] = {1.0, 1};
        }
        const bool any = out.cluster->AggregateGradients(grads, headers, step == 0, true);
        CHECK(any, "samples were processed");
        detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
        // headers: every worker holds the sum
        size_t ns = 0;
        double crit = 0;
        for (size_t r = 0; r < K; ++r)
        {
            ns += 10 + r;
            crit += 1.5 * (double) (r + 1);
        }
        for (size_t r = 0; r < K; ++r)
        {
            CHECK(headers[r].numSamples == ns && std::fabs(headers[r].criterion - crit) < 1e-12, "header sum on worker %zu", r);
            CHECK(headers[r].evalErrors[1].second == K, "eval error denominators");
        }
        if (checkAllWorkersEqual)
            for (size_t r = 1; r < K; ++r)
                for (size_t i = 0; i < shapes.size(); ++i)
                    CHECK(SameBits(*sets[0].ptrs[i], *sets[r].ptrs[i]), "worker %zu, matrix %zu differs from worker 0", r, i);
        out.gradients.emplace_back();
        for (size_t i = 0; i < shapes.size(); ++i)
        {
            auto a = sets[0].ptrs[i]->CopyToArray();
            out.gradients.back().emplace_back(a.get(), a.get() + sets[0].ptrs[i]->GetNumElements());
        }
        out.last = std::move(sets);
    }
    return out;
}

static void VariantsAreBitIdentical()
{
    // (14340 rows: the stripe reduction's register kernel; 110000 rows: taller than any workgroup holds, quantized and reduced
    // by several workgroups per column -- fused where the library says it takes the stripe, else by the reference's call
    // sequence, and a cluster with such a matrix issues its calls worker by worker)
    const Shapes shapes = {{2048, 40}, {429, 37}, {64, 5}, {576, 24}, {1, 9}, {33, 3}, {14340, 6}, {110000, 5}};
    const size_t K = 4;
    for (int nBits : {1, 4})
        for (bool zeroThr : {false, true})
        {
            if (nBits != 1 && zeroThr)
                continue;
            // the reference's arrangement: per-matrix calls, unfused stripe reduction, main stream
            RunResult ref = Run(shapes, K, nBits, zeroThr, true, false, false, false, 3, 4242, true);
            // variants 6 and 7 (fused and batched) issue one call per step for the whole cluster; 8 and 9 are the same two
            // with every worker issuing its own calls
            for (int variant = 1; variant < 10; ++variant)
            {
                const bool useAsync = variant & 1, fused = (variant & 2) || variant >= 8, batched = (variant & 4) || variant >= 8;
                RunResult v = Run(shapes, K, nBits, zeroThr, true, useAsync, fused, batched, 3, 4242, false, variant < 8);
                for (size_t step = 0; step < ref.gradients.size(); ++step)
                    for (size_t i = 0; i < shapes.size(); ++i)
                        CHECK(ref.gradients[step][i].size() == v.gradients[step][i].size() &&
                                  std::memcmp(ref.gradients[step][i].data(), v.gradients[step][i].data(), ref.gradients[step][i].size() * 4) == 0,
                              "bits=%d zeroThr=%d variant=%d step=%zu matrix=%zu", nBits, (int) zeroThr, variant, step, i);
                for (size_t r = 0; r < K; ++r)
                    for (size_t i = 0; i < shapes.size(); ++i)
                    {
                        CHECK(SameBits(ref.cluster->Worker(r).GradientResidual(i), v.cluster->Worker(r).GradientResidual(i)), "gradient residual");
                        const Matrix<float>* a = ref.cluster->Worker(r).StripeResidual(i);
                        const Matrix<float>* b = v.cluster->Worker(r).StripeResidual(i);
                        CHECK((a == nullptr) == (b == nullptr) && (a == nullptr || SameBits(*a, *b)), "stripe residual");
                    }
            }
        }
}

static void AgainstOracle()
{
    const Shapes shapes = {{2048, 24}, {429, 37}, {100, 50}, {64, 3}};
    const size_t K = 8;
    const int steps = 3;
    struct Case { int nBits; bool zeroThr; };
    for (Case c : {Case{1, false}, Case{1, true}, Case{2, false}, Case{4, false}, Case{32, false}})
    {
        RunResult gpu = Run(shapes, K, c.nBits, c.zeroThr, true, true, true, true, steps, 99, true);
        // oracle: one all-reduce per matrix and step, residuals carried
        for (size_t i = 0; i < shapes.size(); ++i)
        {
            const size_t rows = shapes[i].first, cols = shapes[i].second, n = rows * cols;
            const size_t qbytes = oracle_qcol_bytes(c.nBits, rows) * cols;
            std::vector<std::vector<float>> res(K, std::vector<float>(n, 0.0f)), sres(K);
            for (size_t s = 0; s < K; ++s)
            {
                size_t start, len;
                oracle_stripe_range(cols, s, K, &start, &len);
                sres[s].assign(rows * len + 1, 0.0f);
            }
            for (int step = 0; step < steps; ++step)
            {
                std::vector<std::vector<float>> g(K);
                std::vector<std::vector<char>> q(K, std::vector<char>(qbytes));
                std::vector<const float*> gp;
                std::vector<float*> rp, sp;
                std::vector<void*> qp;
                for (size_t r = 0; r < K; ++r)
                {
                    g[r] = Gaussian(n, 0.01f, 99 + 1000 * step + 10 * r + i);
                    gp.push_back(g[r].data());
                    rp.push_back(res[r].data());
                    sp.push_back(sres[r].data());
                    qp.push_back(q[r].data());
                }
                std::vector<char> qagg(qbytes);
                std::vector<float> out(n);
                oracle_allreduce(gp.data(), rp.data(), qp.data(), sp.data(), K, rows, cols, c.nBits, c.zeroThr, qagg.data(), out.data(), 4);
                const std::vector<float>& got = gpu.gradients[step][i];
                if (c.nBits == 32)
                {
                    CHECK(std::memcmp(got.data(), out.data(), n * 4) == 0, "32 bits must reproduce the ordered fp32 sum exactly (matrix %zu)", i);
                    continue;
                }
                // the reference unit test's GPU tolerance: 1e-4 of the value range, at most 0.1 % outliers
                const float tolerance = 0.08f * 8 * 1e-4f;
                size_t bad = 0;
                for (size_t e = 0; e < n; ++e)
                    if (std::fabs(got[e] - out[e]) > tolerance)
                        bad++;
                CHECK(bad <= std::max<size_t>(1, n / 1000), "bits=%d zeroThr=%d matrix %zu step %d: %zu of %zu elements off", c.nBits, (int) c.zeroThr, i, step, bad, n);
            }
        }
    }
}

static void UnquantizedSelfStripe()
{
    // useQuantizationForSelfStripe = false: the owner's own contribution enters the sum unquantized
    // (Source/1BitSGD/AllReduceDistGradAggregator.h:366-375); with 32 bits both settings give the plain sum
    const Shapes shapes = {{128, 16}, {33, 5}};
    RunResult a = Run(shapes, 3, 32, false, false, false, true, false, 2, 7, true);
    RunResult b = Run(shapes, 3, 32, false, true, false, true, false, 2, 7, true);
    for (size_t step = 0; step < a.gradients.size(); ++step)
        for (size_t i = 0; i < shapes.size(); ++i)
            CHECK(a.gradients[step][i] == b.gradients[step][i], "32-bit aggregate independent of self-stripe setting");
    // at 1 bit the two settings differ, and every worker still ends with identical gradients
    RunResult c = Run(shapes, 3, 1, true, false, true, true, true, 2, 7, true);
    RunResult d = Run(shapes, 3, 1, true, true, true, true, true, 2, 7, true);
    CHECK(c.gradients[1][0] != d.gradients[1][0], "self-stripe setting must matter at 1 bit");
}

static void EmptyMinibatchAndReset()
{
    const Shapes shapes = {{256, 12}, {64, 7}};
    const size_t K = 3;
    InProcessCluster<float> cluster(K, 0, 1, true);
    auto step = [&](bool reset, size_t silent, std::vector<WorkerSet>& sets, std::vector<DistGradHeader>& headers) {
        std::vector<std::vector<std::vector<float>>> host(K);
        for (size_t r = 0; r < K; ++r)
            for (size_t i = 0; i < shapes.size(); ++i)
                host[r].push_back(Gaussian(shapes[i].first * shapes[i].second, 0.01f, 5 + 10 * r + i));
        sets = MakeGradients(shapes, K, host);
        std::vector<std::vector<Matrix<float>*>> grads;
        headers.clear();
        for (size_t r = 0; r < K; ++r)
        {
            grads.push_back(sets[r].ptrs);
            headers.emplace_back(1);
            headers.back().numSamples = (r == silent) ? 0 : 4;
        }
        cluster.AggregateGradients(grads, headers, reset);
        detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
    };
    std::vector<WorkerSet> s1, s2, s3;
    std::vector<DistGradHeader> h1, h2, h3;
    step(true, K, s1, h1);  // everybody has samples
    step(true, K, s2, h2);  // same inputs after a reset: identical result, i.e. no residual survived the reset
    for (size_t i = 0; i < shapes.size(); ++i)
        CHECK(SameBits(*s1[0].ptrs[i], *s2[0].ptrs[i]), "resetState must clear every residual");
    step(true, 1, s3, h3);  // worker 1 saw no samples: its gradients are zeroed before quantization
    CHECK(h3[0].numSamples == 8, "header sum with a silent worker");
    for (size_t i = 0; i < shapes.size(); ++i)
        CHECK(!SameBits(*s1[0].ptrs[i], *s3[0].ptrs[i]), "a silent worker changes the aggregate");
}

// The double-buffered aggregation (Source/1BitSGD/AllReduceDistGradAggregator.h:155-225): call t hands back what a
// synchronous aggregator produced for the input of call t - 1, bit for bit, and zeros the first time; without resetState
// and with no samples in the header that comes back, nothing is started.
static void BufferedAggregation()
{
    const Shapes shapes = {{2048, 24}, {429, 37}, {64, 5}};
    const size_t K = 4;
    const int steps = 4;
    InProcessCluster<float> sync(K, 0, 1, false), buffered(K, 0, 1, false);
    std::vector<std::vector<std::vector<float>>> expected; // [step][matrix] of worker 0 from the synchronous cluster
    std::vector<size_t> expectedSamples;
    for (int step = 0; step <= steps; ++step)
    {
        std::vector<std::vector<std::vector<float>>> host(K);
        for (size_t r = 0; r < K; ++r)
            for (size_t i = 0; i < shapes.size(); ++i)
                host[r].push_back(Gaussian(shapes[i].first * shapes[i].second, 0.01f, 5150 + 1000 * step + 10 * r + i));
        std::vector<WorkerSet> a = MakeGradients(shapes, K, host), b = MakeGradients(shapes, K, host);
        std::vector<std::vector<Matrix<float>*>> ga, gb;
        std::vector<DistGradHeader> ha, hb;
        for (size_t r = 0; r < K; ++r)
        {
            ga.push_back(a[r].ptrs);
            gb.push_back(b[r].ptrs);
            ha.emplace_back(1);
            ha.back().numSamples = 7 + r + step;
            hb.push_back(ha.back());
        }
        if (step < steps)
        {
            sync.AggregateGradients(ga, ha, step == 0, true);
            detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
            expected.emplace_back();
            for (size_t i = 0; i < shapes.size(); ++i)
            {
                auto x = a[0].ptrs[i]->CopyToArray();
                expected.back().emplace_back(x.get(), x.get() + a[0].ptrs[i]->GetNumElements());
            }
            expectedSamples.push_back(ha[0].numSamples);
        }
        const bool started = buffered.AggregateGradientsBuffered(gb, hb, step == 0);
        CHECK(started, "step %d: aggregation started", step);
        for (size_t r = 0; r < K; ++r)
            for (size_t i = 0; i < shapes.size(); ++i)
            {
                auto x = b[r].ptrs[i]->CopyToArray();
                const size_t n = b[r].ptrs[i]->GetNumElements();
                if (step == 0)
                {
                    bool zero = true;
                    for (size_t e = 0; e < n; ++e)
                        zero = zero && x[e] == 0.0f;
                    CHECK(zero && hb[r].numSamples == 0, "the first call hands back zeros");
                }
                else
                    CHECK(std::memcmp(x.get(), expected[step - 1][i].data(), n * 4) == 0 && hb[r].numSamples == expectedSamples[step - 1],
                          "step %d worker %zu matrix %zu: the previous call's aggregate", step, r, i);
            }
    }
    buffered.WaitForPendingAggregation();

    // nothing starts without resetState while the header that comes back has no samples; the gradients are exchanged all the same
    InProcessCluster<float> idle(K, 0, 1, false);
    std::vector<std::vector<std::vector<float>>> host(K);
    for (size_t r = 0; r < K; ++r)
        for (size_t i = 0; i < shapes.size(); ++i)
            host[r].push_back(Gaussian(shapes[i].first * shapes[i].second, 0.01f, 77 + 10 * r + i));
    std::vector<WorkerSet> first = MakeGradients(shapes, K, host), second = MakeGradients(shapes, K, host);
    std::vector<std::vector<Matrix<float>*>> g1, g2;
    std::vector<DistGradHeader> h1, h2;
    for (size_t r = 0; r < K; ++r)
    {
        g1.push_back(first[r].ptrs);
        g2.push_back(second[r].ptrs);
        h1.emplace_back(1);
        h1.back().numSamples = 3;
        h2.emplace_back(1);
        h2.back().numSamples = 4;
    }
    CHECK(!idle.AggregateGradientsBuffered(g1, h1, false), "no aggregation without reset and without samples coming back");
    CHECK(idle.AggregateGradientsBuffered(g2, h2, false), "the header coming back now has samples");
    CHECK(h2[0].numSamples == 3, "the header handed back is the first call's own");
    auto x = second[0].ptrs[0]->CopyToArray();
    CHECK(std::memcmp(x.get(), host[0][0].data(), host[0][0].size() * 4) == 0, "and so are the gradients: never aggregated");
    idle.WaitForPendingAggregation();
}

// The double instantiation (the reference's end-to-end 1-bit tests run in double precision): the reference's arrangement
// of calls against fused stripe reduction + batched calls, bit for bit, over carried steps (tile and 256-thread register kernels up to 6144 rows,
// 1024-thread register kernels above; 52000 rows are too tall for the fused reduction and keep the call sequence).
static void DoublePrecisionVariantsAreBitIdentical()
{
    const Shapes shapes = {{2048, 12}, {429, 17}, {64, 5}, {1, 9}, {4096, 4}, {147, 3}, {6000, 6}, {7000, 4}, {52000, 3}};
    const size_t K = 3;
    for (int nBits : {1, 8})
    {
        std::vector<std::vector<std::vector<double>>> results[2]; // [arrangement][step][matrix] of worker 0
        for (int arrangement = 0; arrangement < 2; ++arrangement)
        {
            InProcessCluster<double>::Options opt;
            opt.useFusedStripeReduce = arrangement == 1;
            opt.useBatchedCalls = arrangement == 1;
            InProcessCluster<double> cluster(K, 0, nBits, false, true, arrangement == 1, opt);
            for (int step = 0; step < 3; ++step)
            {
                std::vector<std::vector<std::unique_ptr<Matrix<double>>>> owned(K);
                std::vector<std::vector<Matrix<double>*>> grads(K);
                std::vector<DistGradHeader> headers;
                for (size_t r = 0; r < K; ++r)
                {
                    for (size_t i = 0; i < shapes.size(); ++i)
                    {
                        const std::vector<float> f = Gaussian(shapes[i].first * shapes[i].second, 0.01f, 777 + 1000 * step + 10 * r + i);
                        const std::vector<double> d(f.begin(), f.end());
                        owned[r].emplace_back(new Matrix<double>(shapes[i].first, shapes[i].second, 0));
                        owned[r].back()->SetValue(d.data());
                        grads[r].push_back(owned[r].back().get());
                    }
                    headers.emplace_back(1);
                    headers.back().numSamples = 5 + r;
                }
                cluster.AggregateGradients(grads, headers, step == 0, true);
                detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
                results[arrangement].emplace_back();
                for (size_t i = 0; i < shapes.size(); ++i)
                {
                    auto a = grads[0][i]->CopyToArray();
                    results[arrangement].back().emplace_back(a.get(), a.get() + grads[0][i]->GetNumElements());
                    for (size_t r = 1; r < K; ++r)
                    {
                        auto b = grads[r][i]->CopyToArray();
                        CHECK(std::memcmp(a.get(), b.get(), grads[0][i]->GetNumElements() * sizeof(double)) == 0,
                              "double: worker %zu, matrix %zu differs from worker 0", r, i);
                    }
                }
            }
        }
        for (size_t step = 0; step < results[0].size(); ++step)
            for (size_t i = 0; i < shapes.size(); ++i)
                CHECK(std::memcmp(results[0][step][i].data(), results[1][step][i].data(), results[0][step][i].size() * sizeof(double)) == 0,
                      "double: bits=%d step=%zu matrix=%zu: fused + batched differs from the reference's arrangement", nBits, step, i);
    }
}

// syncStatsTrace = 2: every second aggregation reports its time on stderr (the reference's wording).
static void SyncStatsTrace()
{
    InProcessCluster<float>::Options opt;
    opt.syncStatsTrace = 2;
    InProcessCluster<float> cluster(2, 0, 1, false, true, false, opt);
    FILE* saved = stderr;
    FILE* f = std::tmpfile();
    CHECK(f != nullptr, "tmpfile");
    if (f == nullptr)
        return;
    stderr = f;
    for (int step = 0; step < 5; ++step)
    {
        std::vector<std::unique_ptr<Matrix<float>>> owned;
        std::vector<std::vector<Matrix<float>*>> grads(2);
        std::vector<DistGradHeader> headers;
        for (size_t r = 0; r < 2; ++r)
        {
            owned.emplace_back(new Matrix<float>(64, 8, 0));
            owned.back()->SetValue(0.01f * (float) (r + 1));
            grads[r].push_back(owned.back().get());
            headers.emplace_back(1);
            headers.back().numSamples = 4;
        }
        cluster.AggregateGradients(grads, headers, step == 0, true);
    }
    stderr = saved;
    std::rewind(f);
    int lines = 0;
    char buf[256];
    while (std::fgets(buf, sizeof buf, f) != nullptr)
        if (std::strstr(buf, "Actual gradient aggregation time: ") != nullptr)
            lines++;
    std::fclose(f);
    CHECK(lines == 3, "aggregations 0, 2 and 4 are reported, got %d lines", lines);
}

// traceLevel = 3: the 3 x 3 corners of the original gradients, of the packed stripes sent and received and of the aggregated
// gradients go to stderr, in the reference's wording; the aggregation itself gives the bytes it gives without them.
static void DebugPeeks()
{
    const size_t K = 2;
    std::vector<std::vector<float>> results[2];
    std::string text;
    for (int traced = 0; traced < 2; ++traced)
    {
        InProcessCluster<float>::Options opt;
        opt.traceLevel = traced ? 3 : 0;
        InProcessCluster<float> cluster(K, 0, 1, false, true, false, opt);
        FILE* saved = stderr;
        FILE* f = std::tmpfile();
        CHECK(f != nullptr, "tmpfile");
        if (f == nullptr)
            return;
        stderr = f;
        std::vector<std::unique_ptr<Matrix<float>>> owned;
        std::vector<std::vector<Matrix<float>*>> grads(K);
        std::vector<DistGradHeader> headers;
        for (size_t r = 0; r < K; ++r)
        {
            for (size_t i = 0; i < 2; ++i)
            {
                const size_t rows = i == 0 ? 64 : 2, cols = i == 0 ? 8 : 5;
                owned.emplace_back(new Matrix<float>(rows, cols, 0));
                owned.back()->SetValue(Gaussian(rows * cols, 0.01f, 77 + 10 * r + i).data());
                grads[r].push_back(owned.back().get());
            }
            headers.emplace_back(1);
            headers.back().numSamples = 4;
        }
        cluster.AggregateGradients(grads, headers, true, true);
        detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
        stderr = saved;
        std::rewind(f);
        char buf[512];
        while (std::fgets(buf, sizeof buf, f) != nullptr)
            if (traced)
                text += buf;
            else
                CHECK(false, "output without tracing: %s", buf);
        std::fclose(f);
        for (auto* g : grads[0])
        {
            auto a = g->CopyToArray();
            results[traced].emplace_back(a.get(), a.get() + g->GetNumElements());
        }
    }
    for (size_t i = 0; i < results[0].size(); ++i)
        CHECK(results[0][i].size() == results[1][i].size() &&
                  std::memcmp(results[0][i].data(), results[1][i].data(), results[0][i].size() * sizeof(float)) == 0,
              "matrix %zu: the traced aggregation gives other bytes", i);
    auto count = [&](const char* what) {
        int n = 0;
        for (size_t at = text.find(what); at != std::string::npos; at = text.find(what, at + 1))
            n++;
        return n;
    };
    CHECK(count("MPI Rank: 0, Original Gradient Matrix No. 0 (64, 8) [0:2, 0:2] ######") == 1, "original gradient of rank 0");
    CHECK(count("MPI Rank: 1, Original Gradient Matrix No. 1 (2, 5) [0:1, 0:2] ######") == 1, "a matrix of two rows is peeked at two rows");
    CHECK(count("Sending Gradient Matrix No.") == 4, "every rank sends one slice of every matrix to the other: %d", count("Sending Gradient Matrix No."));
    CHECK(count("Received Gradient Matrix No.") == 4, "and receives one: %d", count("Received Gradient Matrix No."));
    CHECK(count("Aggregated Gradient Matrix No.") == 4, "aggregated gradients: %d", count("Aggregated Gradient Matrix No."));
    CHECK(count("Lower=") >= 8 && count("------ Print Range (0:2, 0:2) ------") >= 1, "packed stripes are printed with their column bounds");
}

int main()
{
    try
    {
        struct T { const char* name; void (*fn)(); };
        const T tests[] = {{"QuantizedAllReduceVariantsBitIdentical", VariantsAreBitIdentical}, {"QuantizedAllReduceAgainstOracle", AgainstOracle},
                           {"QuantizedAllReduceUnquantizedSelfStripe", UnquantizedSelfStripe}, {"QuantizedAllReduceEmptyMinibatchAndReset", EmptyMinibatchAndReset},
                           {"QuantizedAllReduceBufferedAggregation", BufferedAggregation},
                           {"QuantizedAllReduceDoublePrecision", DoublePrecisionVariantsAreBitIdentical},
                           {"QuantizedAllReduceSyncStatsTrace", SyncStatsTrace}, {"QuantizedAllReduceDebugPeeks", DebugPeeks}};
        for (const T& t : tests)
        {
            const int before = g_failures;
            t.fn();
            std::printf("Test case AggregatorSuite/%s %s\n", t.name, g_failures != before ? "has FAILED" : "has passed");
            std::fflush(stdout);
        }
    }
    catch (const std::exception& e)
    {
        std::fprintf(stderr, "unexpected exception: %s\n", e.what());
        return 2;
    }
    return g_failures ? 1 : 0;
}
