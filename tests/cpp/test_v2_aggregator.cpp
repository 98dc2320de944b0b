// Tests of the aggregator over the v2 communicator (cntk_amd/cpp/V2AllReduceDistGradAggregator.h) with K workers in one
// process on one GPU.
//
//   * against the v1 aggregator (cntk_amd/cpp/AllReduceDistGradAggregator.h) on the same gradients and headers, several
//     minibatches in a row so that both kinds of residue carry over: the same bytes in every worker's gradients and
//     the same aggregated header (float at 1 and 2 bits, double at 1 bit);
//   * the header as doubles: what is packed comes back, with several evaluation nodes, and the aggregate of K headers
//     is their sum in every field;
//   * a worker whose header saw no samples contributes zeros, whatever its gradient matrices held;
//   * reset: after resetState the same gradients aggregate to the same bytes as the first time;
//   * double buffering: a call returns the aggregate of what the call before it was given (zeros and a cleared header
//     the first time), starts aggregating only after a call that saw samples or on a reset, and a reset while an
//     aggregation is pending is refused with the reference's message.
#include "../../cntk_amd/cpp/V2AllReduceDistGradAggregator.h"

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

template <class ElemType>
struct GradientSets // K workers' gradient matrices
{
    std::vector<std::vector<std::unique_ptr<Matrix<ElemType>>>> owned;
    std::vector<std::vector<Matrix<ElemType>*>> pointers;

    GradientSets(const Shapes& shapes, size_t K) : owned(K), pointers(K)
    {
        for (size_t r = 0; r < K; ++r)
            for (const auto& s : shapes)
            {
                owned[r].emplace_back(new Matrix<ElemType>(s.first, s.second, 0));
                pointers[r].push_back(owned[r].back().get());
            }
    }
    void Fill(unsigned long seed)
    {
        for (size_t r = 0; r < owned.size(); ++r)
            for (size_t i = 0; i < owned[r].size(); ++i)
            {
                std::mt19937_64 rng(seed + 100 * r + i);
                std::normal_distribution<double> d(0.0, 0.01);
                std::vector<ElemType> a(owned[r][i]->GetNumElements());
                for (auto& x : a)
                    x = (ElemType) d(rng);
                owned[r][i]->SetValue(a.data());
            }
    }
    std::vector<ElemType> Host(size_t r, size_t i) const
    {
        auto a = pointers[r][i]->CopyToArray();
        return std::vector<ElemType>(a.get(), a.get() + pointers[r][i]->GetNumElements());
    }
};

template <class ElemType>
static bool SameBits(const std::vector<ElemType>& a, const std::vector<ElemType>& b)
{
    return a.size() == b.size() && (a.empty() || std::memcmp(a.data(), b.data(), a.size() * sizeof(ElemType)) == 0);
}

static std::vector<DistGradHeader> MakeHeaders(size_t K, int numEvalNode, int step)
{
    std::vector<DistGradHeader> headers;
    for (size_t r = 0; r < K; ++r)
    {
        headers.emplace_back(numEvalNode);
        DistGradHeader& h = headers.back();
        h.numSamples = 16 + r + (size_t) step;
        h.numSamplesWithLabel = 15 + r;
        h.criterion = 0.5 * (double) (r + 1) + (double) step;
        for (int e = 0; e < numEvalNode; ++e)
            h.evalErrors[(size_t) e] = {0.25 * (double) (r + 1) + e, (size_t) (7 + r + (size_t) e)};
    }
    return headers;
}

static bool SameHeader(const DistGradHeader& a, const DistGradHeader& b)
{
    return a.numSamples == b.numSamples && a.numSamplesWithLabel == b.numSamplesWithLabel && a.criterion == b.criterion && a.evalErrors == b.evalErrors;
}

template <class ElemType>
static void EqualsV1(int nBits, const Shapes& shapes, size_t K)
{
    InProcessCluster<ElemType> v1(K, 0, nBits, false, true, true);
    InProcessV2Aggregators<ElemType> v2(K, false, true, (size_t) nBits, false);
    GradientSets<ElemType> a(shapes, K), b(shapes, K);
    for (int step = 0; step < 3; ++step)
    {
        a.Fill(31 * step + 5);
        b.Fill(31 * step + 5);
        auto ha = MakeHeaders(K, 2, step), hb = MakeHeaders(K, 2, step);
        const bool ra = v1.AggregateGradients(a.pointers, ha, step == 0, true);
        const bool rb = v2.AggregateGradients(b.pointers, hb, step == 0);
        detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
        CHECK(ra == rb && rb, "return value: bits %d step %d", nBits, step);
        for (size_t r = 0; r < K; ++r)
        {
            CHECK(SameHeader(ha[r], hb[r]), "header: bits %d step %d worker %zu", nBits, step, r);
            for (size_t i = 0; i < shapes.size(); ++i)
                CHECK(SameBits(a.Host(r, i), b.Host(r, i)), "v2 aggregator != v1 aggregator: bits %d step %d worker %zu gradient %zu", nBits, step, r, i);
        }
    }
}

static void EqualsV1Float()
{
    EqualsV1<float>(1, {{2048, 24}, {429, 37}, {100, 50}, {64, 3}, {9304, 8}}, 8);
    EqualsV1<float>(2, {{512, 33}, {77, 5}}, 3);
}
static void EqualsV1Double()
{
    EqualsV1<double>(1, {{1024, 17}, {300, 40}}, 4);
}

static void HeaderAsDoubles()
{
    DistGradHeader h(3);
    h.numSamples = 123456789;
    h.numSamplesWithLabel = 123450000;
    h.criterion = -3.25;
    h.evalErrors = {{1.5, 10}, {0.0, 0}, {7.125, 4000000000ull}};
    const auto packed = V2AllReduceDistGradAggregator<float>::PackHeader(h);
    CHECK(packed.size() == 9, "3 + 2 per evaluation node, got %zu", packed.size());
    CHECK(packed[0] == -3.25 && packed[1] == 123456789.0 && packed[2] == 123450000.0 && packed[3] == 1.5 && packed[4] == 10.0 && packed[8] == 4e9,
          "order of the fields");
    DistGradHeader back(3);
    V2AllReduceDistGradAggregator<float>::UnpackHeader(packed, back);
    CHECK(SameHeader(h, back), "round trip");
    DistGradHeader other(2);
    bool threw = false;
    try
    {
        V2AllReduceDistGradAggregator<float>::UnpackHeader(packed, other);
    }
    catch (const std::logic_error&)
    {
        threw = true;
    }
    CHECK(threw, "a header of another size is refused");

    // the aggregate of K headers
    const size_t K = 5;
    InProcessV2Aggregators<float> v2(K, false, true, 1, false);
    GradientSets<float> g({{64, 10}}, K);
    g.Fill(3);
    auto headers = MakeHeaders(K, 2, 0);
    DistGradHeader sum(2);
    for (size_t r = 0; r < K; ++r)
        sum.Aggregate(headers[r], r != 0);
    v2.AggregateGradients(g.pointers, headers, true);
    for (size_t r = 0; r < K; ++r)
        CHECK(SameHeader(headers[r], sum), "aggregated header on worker %zu", r);
}

static void WorkerWithoutSamples()
{
    const Shapes shapes = {{256, 12}, {50, 9}};
    const size_t K = 4;
    InProcessV2Aggregators<float> idle(K, false, true, 1, false), zeros(K, false, true, 1, false);
    GradientSets<float> a(shapes, K), b(shapes, K);
    a.Fill(11);
    b.Fill(11);
    for (auto* m : b.pointers[2])
        m->SetValue(0.0f);
    auto ha = MakeHeaders(K, 1, 0), hb = MakeHeaders(K, 1, 0);
    ha[2].Clear(); // worker 2 saw nothing: its matrices hold leftovers
    hb[2].Clear();
    idle.AggregateGradients(a.pointers, ha, true);
    zeros.AggregateGradients(b.pointers, hb, true);
    for (size_t r = 0; r < K; ++r)
        for (size_t i = 0; i < shapes.size(); ++i)
            CHECK(SameBits(a.Host(r, i), b.Host(r, i)), "worker %zu gradient %zu", r, i);

    // nobody saw anything: the call says so
    InProcessV2Aggregators<float> nobody(K, false, true, 1, false);
    std::vector<DistGradHeader> none;
    for (size_t r = 0; r < K; ++r)
        none.emplace_back(1);
    CHECK(!nobody.AggregateGradients(a.pointers, none, true), "no samples anywhere");
}

static void ResetClearsResidues()
{
    const Shapes shapes = {{1024, 9}, {33, 20}};
    const size_t K = 3;
    InProcessV2Aggregators<float> v2(K, false, true, 1, false);
    GradientSets<float> g(shapes, K);
    std::vector<std::vector<float>> first;
    for (int step = 0; step < 3; ++step)
    {
        g.Fill(77); // the same gradients every time
        auto h = MakeHeaders(K, 1, 0);
        v2.AggregateGradients(g.pointers, h, step != 1);
        std::vector<std::vector<float>> now;
        for (size_t i = 0; i < shapes.size(); ++i)
            now.push_back(g.Host(0, i));
        if (step == 0)
            first = now;
        else if (step == 1) // residues carried over: another result
            CHECK(!SameBits(now[0], first[0]), "the second minibatch used the first one's residues");
        else
            for (size_t i = 0; i < shapes.size(); ++i)
                CHECK(SameBits(now[i], first[i]), "after a reset, gradient %zu", i);
    }
}

static void DoubleBuffered()
{
    const Shapes shapes = {{2048, 16}, {100, 30}};
    const size_t K = 4;
    InProcessV2Aggregators<float> sync(K, false, true, 1, false), async(K, false, true, 1, true);
    GradientSets<float> s(shapes, K), a(shapes, K);
    std::vector<std::vector<std::vector<float>>> expected; // [call][worker * gradients + i]
    std::vector<std::vector<DistGradHeader>> expectedHeaders;
    const int calls = 4;
    for (int call = 0; call < calls; ++call)
    {
        s.Fill(900 + call);
        auto hs = MakeHeaders(K, 1, call);
        sync.AggregateGradients(s.pointers, hs, call == 0);
        expected.emplace_back();
        for (size_t r = 0; r < K; ++r)
            for (size_t i = 0; i < shapes.size(); ++i)
                expected.back().push_back(s.Host(r, i));
        expectedHeaders.push_back(hs);
    }
    for (int call = 0; call <= calls; ++call)
    {
        a.Fill(900 + call);
        auto ha = MakeHeaders(K, 1, call);
        const bool started = async.AggregateGradients(a.pointers, ha, call == 0);
        CHECK(started, "call %d starts an aggregation", call);
        if (call == 0)
        {
            for (size_t r = 0; r < K; ++r)
            {
                CHECK(ha[r].numSamples == 0 && ha[r].criterion == 0.0, "first call: a cleared header");
                for (size_t i = 0; i < shapes.size(); ++i)
                {
                    const auto host = a.Host(r, i);
                    bool allZero = true;
                    for (float x : host)
                        allZero = allZero && x == 0.0f;
                    CHECK(allZero, "first call: zeros");
                }
            }
            continue;
        }
        for (size_t r = 0; r < K; ++r)
        {
            CHECK(SameHeader(ha[r], expectedHeaders[(size_t) call - 1][r]), "call %d worker %zu: the header of the call before", call, r);
            for (size_t i = 0; i < shapes.size(); ++i)
                CHECK(SameBits(a.Host(r, i), expected[(size_t) call - 1][r * shapes.size() + i]), "call %d worker %zu gradient %zu: the aggregate of the call before",
                      call, r, i);
        }
    }
    // a reset while the last call's aggregation has not been waited for
    {
        auto ha = MakeHeaders(K, 1, 0);
        bool threw = false;
        try
        {
            async.AggregateGradients(a.pointers, ha, true);
        }
        catch (const std::logic_error& e)
        {
            threw = std::strstr(e.what(), "Unexpected pending async gradient aggregation") != nullptr;
        }
        CHECK(threw, "reset with an aggregation pending");
        async.WaitForPendingAggregation();
    }
    // a call after one that saw no samples anywhere starts nothing
    {
        InProcessV2Aggregators<float> quiet(K, false, true, 1, true);
        std::vector<DistGradHeader> none;
        for (size_t r = 0; r < K; ++r)
            none.emplace_back(1);
        a.Fill(5);
        CHECK(quiet.AggregateGradients(a.pointers, none, true), "first call: reset starts an aggregation");
        quiet.WaitForPendingAggregation();
        std::vector<DistGradHeader> again;
        for (size_t r = 0; r < K; ++r)
            again.emplace_back(1);
        CHECK(!quiet.AggregateGradients(a.pointers, again, false), "the aggregate that came back saw no samples: nothing started");
    }
}

int main()
{
    try
    {
        struct T { const char* name; void (*fn)(); };
        const T tests[] = {{"EqualsV1AggregatorFloat", EqualsV1Float}, {"EqualsV1AggregatorDouble", EqualsV1Double}, {"HeaderAsDoubles", HeaderAsDoubles},
                           {"WorkerWithoutSamples", WorkerWithoutSamples}, {"ResetClearsResidues", ResetClearsResidues}, {"DoubleBuffered", DoubleBuffered}};
        for (const T& t : tests)
        {
            const int before = g_failures;
            t.fn();
            std::printf("Test case V2AggregatorSuite/%s %s\n", t.name, g_failures != before ? "has FAILED" : "has passed");
            std::fflush(stdout);
        }
    }
    catch (const std::exception& e)
    {
        std::fprintf(stderr, "unexpected exception: %s\n", e.what());
        return 2;
    }
    return g_failures == 0 ? 0 : 1;
}
