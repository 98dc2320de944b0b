// Tests of the v2 communicator's call shape (cntk_amd/cpp/QuantizedDistributedCommunicator.h) with K workers in one
// process on one GPU.
//
//   * out-of-place against in-place: a first call that gets empty residue lists (the communicator allocates an input and
//     an output residue per value) followed by a call on the new residues gives, bit for bit, what two in-place calls on
//     aliased buffers give -- outputs, value residues and stripe residues; the out-of-place call with the fused stripe
//     reduction leaves its inputs untouched;
//   * the v1 aggregator (cntk_amd/cpp/AllReduceDistGradAggregator.h) on the same gradients: the same bytes;
//   * the fused stripe reduction against the reference's sequence of calls: the same bytes;
//   * float and double by the values' type; a list that mixes them is refused with the reference's message; a
//     communicator of one worker hands its inputs back.
#include "../../cntk_amd/cpp/QuantizedDistributedCommunicator.h"

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
typedef InProcessCommunicators::PerWorker PerWorker;

template <class ElemType>
static std::vector<ElemType> Gaussian(size_t n, double sigma, unsigned long seed)
{
    std::mt19937_64 rng(seed);
    std::normal_distribution<double> d(0.0, sigma);
    std::vector<ElemType> a(n);
    for (auto& x : a)
        x = (ElemType) d(rng);
    return a;
}

template <class ElemType>
static PerWorker MakeValues(const Shapes& shapes, size_t K, unsigned long seed)
{
    PerWorker values(K);
    for (size_t r = 0; r < K; ++r)
        for (size_t i = 0; i < shapes.size(); ++i)
        {
            auto v = std::make_shared<NDArrayView>(AsDataType<ElemType>(), shapes[i].first, shapes[i].second, 0);
            v->template GetWritableMatrix<ElemType>()->SetValue(Gaussian<ElemType>(shapes[i].first * shapes[i].second, 0.01, seed + 10 * r + i).data());
            values[r].push_back(v);
        }
    return values;
}

template <class ElemType>
static PerWorker MakeEmptyLike(const PerWorker& like)
{
    PerWorker out(like.size());
    for (size_t r = 0; r < like.size(); ++r)
        for (const auto& v : like[r])
            out[r].push_back(std::make_shared<NDArrayView>(AsDataType<ElemType>(), v->GetNumRows(), v->GetNumCols(), 0));
    return out;
}

template <class ElemType>
static std::vector<ElemType> Host(const NDArrayViewPtr& v)
{
    auto m = v->template GetWritableMatrix<ElemType>();
    auto a = m->CopyToArray();
    return std::vector<ElemType>(a.get(), a.get() + m->GetNumElements());
}

template <class ElemType>
static bool SameBits(const NDArrayViewPtr& a, const NDArrayViewPtr& b)
{
    if (!a || !b)
        return !a && !b;
    auto x = Host<ElemType>(a), y = Host<ElemType>(b);
    return x.size() == y.size() && std::memcmp(x.data(), y.data(), x.size() * sizeof(ElemType)) == 0;
}

template <class ElemType>
static void OutOfPlaceEqualsAliased(int nBits, bool zeroThr, bool fused)
{
    // (14340 rows: the register kernels; 33 x 3 on 4 workers: a worker without a stripe)
    const Shapes shapes = {{2048, 40}, {429, 37}, {64, 5}, {33, 3}, {14340, 6}};
    const size_t K = 4;
    QuantizedCommunicator::Options opt;
    opt.useFusedStripeReduce = fused;
    detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");

    // A: first call out of place with empty residue lists, second call on the residues the first one produced
    InProcessCommunicators a(K, zeroThr, true, (size_t) nBits, opt);
    PerWorker aIn1 = MakeValues<ElemType>(shapes, K, 100), aOut1 = MakeEmptyLike<ElemType>(aIn1);
    PerWorker aRes(K), aStripe(K), aNewRes(K), aNewStripe(K);
    std::vector<std::vector<std::vector<ElemType>>> before(K);
    for (size_t r = 0; r < K; ++r)
        for (auto& v : aIn1[r])
            before[r].push_back(Host<ElemType>(v));
    a.QuantizedAggregate(aIn1, aRes, aStripe, aOut1, aNewRes, aNewStripe);
    detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
    for (size_t r = 0; r < K; ++r)
    {
        CHECK(aRes[r].size() == shapes.size() && aNewRes[r].size() == shapes.size(), "residues were allocated");
        for (size_t i = 0; i < shapes.size(); ++i)
        {
            CHECK(aRes[r][i] && aNewRes[r][i] && aRes[r][i] != aNewRes[r][i], "an input and an output residue per value");
            const bool owns = AllReduceDistGradAggregator<ElemType>::GetStripeForNode(shapes[i].second, r, K).m_numCols > 0;
            CHECK((aStripe[r][i] != nullptr) == owns && (aNewStripe[r][i] != nullptr) == owns, "stripe residues only where a stripe is owned");
            if (fused)
            {
                auto now = Host<ElemType>(aIn1[r][i]);
                CHECK(std::memcmp(now.data(), before[r][i].data(), now.size() * sizeof(ElemType)) == 0, "input value untouched");
            }
            // the input residues were zero and stay zero
            for (ElemType x : Host<ElemType>(aRes[r][i]))
                if (x != 0)
                {
                    CHECK(false, "input residue modified");
                    break;
                }
        }
    }
    // B: in place from the start
    InProcessCommunicators b(K, zeroThr, true, (size_t) nBits, opt);
    PerWorker bIn1 = MakeValues<ElemType>(shapes, K, 100), bRes(K), bStripe(K);
    b.QuantizedAggregateInPlace(bIn1, bRes, bStripe);
    detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
    for (size_t r = 0; r < K; ++r)
        for (size_t i = 0; i < shapes.size(); ++i)
        {
            CHECK(SameBits<ElemType>(aOut1[r][i], bIn1[r][i]), "first call: output, worker %zu value %zu", r, i);
            CHECK(SameBits<ElemType>(aNewRes[r][i], bRes[r][i]), "first call: value residue, worker %zu value %zu", r, i);
            CHECK(SameBits<ElemType>(aNewStripe[r][i], bStripe[r][i]), "first call: stripe residue, worker %zu value %zu", r, i);
            CHECK(SameBits<ElemType>(aOut1[0][i], aOut1[r][i]), "all workers hold the same aggregate");
        }
    // second call: A goes on in place on the residues its first call wrote
    PerWorker aIn2 = MakeValues<ElemType>(shapes, K, 200);
    a.QuantizedAggregateInPlace(aIn2, aNewRes, aNewStripe);
    PerWorker bIn2 = MakeValues<ElemType>(shapes, K, 200);
    b.QuantizedAggregateInPlace(bIn2, bRes, bStripe);
    detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
    for (size_t r = 0; r < K; ++r)
        for (size_t i = 0; i < shapes.size(); ++i)
        {
            CHECK(SameBits<ElemType>(aIn2[r][i], bIn2[r][i]), "second call: output, worker %zu value %zu", r, i);
            CHECK(SameBits<ElemType>(aNewRes[r][i], bRes[r][i]), "second call: value residue, worker %zu value %zu", r, i);
            CHECK(SameBits<ElemType>(aNewStripe[r][i], bStripe[r][i]), "second call: stripe residue, worker %zu value %zu", r, i);
        }
}

static void OutOfPlaceFloat()
{
    OutOfPlaceEqualsAliased<float>(1, false, true);
    OutOfPlaceEqualsAliased<float>(1, true, false);
    OutOfPlaceEqualsAliased<float>(4, false, true);
}

static void OutOfPlaceDouble()
{
    OutOfPlaceEqualsAliased<double>(1, false, true);
    OutOfPlaceEqualsAliased<double>(2, false, false);
}

// the same gradients through the v1 aggregator and through the communicator, fused and as the reference's call sequence
static void EqualsAggregatorAndCallSequence()
{
    const Shapes shapes = {{2048, 24}, {429, 37}, {100, 50}, {64, 3}, {9304, 8}};
    const size_t K = 8;
    for (int nBits : {1, 2})
    {
        InProcessCluster<float> cluster(K, 0, nBits, false, true, true);
        InProcessCommunicators fused(K, false, true, (size_t) nBits);
        QuantizedCommunicator::Options seq;
        seq.useFusedStripeReduce = false;
        InProcessCommunicators sequence(K, false, true, (size_t) nBits, seq);
        PerWorker fRes(K), fStripe(K), sRes(K), sStripe(K);
        for (int step = 0; step < 3; ++step)
        {
            PerWorker fIn = MakeValues<float>(shapes, K, 1000 * step + 7), sIn = MakeValues<float>(shapes, K, 1000 * step + 7);
            PerWorker cIn = MakeValues<float>(shapes, K, 1000 * step + 7);
            std::vector<std::vector<Matrix<float>*>> grads(K);
            std::vector<DistGradHeader> headers;
            for (size_t r = 0; r < K; ++r)
            {
                for (auto& v : cIn[r])
                    grads[r].push_back(v->GetWritableMatrix<float>().get());
                headers.emplace_back(1);
                headers.back().numSamples = 16;
            }
            cluster.AggregateGradients(grads, headers, step == 0, true);
            fused.QuantizedAggregateInPlace(fIn, fRes, fStripe);
            sequence.QuantizedAggregateInPlace(sIn, sRes, sStripe);
            detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
            for (size_t r = 0; r < K; ++r)
                for (size_t i = 0; i < shapes.size(); ++i)
                {
                    CHECK(SameBits<float>(fIn[r][i], cIn[r][i]), "communicator != aggregator: bits %d step %d worker %zu value %zu", nBits, step, r, i);
                    CHECK(SameBits<float>(fIn[r][i], sIn[r][i]), "fused != call sequence: bits %d step %d worker %zu value %zu", nBits, step, r, i);
                    CHECK(SameBits<float>(fRes[r][i], sRes[r][i]) && SameBits<float>(fStripe[r][i], sStripe[r][i]), "residues, fused != call sequence");
                }
        }
    }
}

static void TypesAndTrivialCases()
{
    // mixed element types
    InProcessCommunicators two(2, false, true, 1);
    PerWorker mixed(2), res(2), stripe(2);
    for (size_t r = 0; r < 2; ++r)
    {
        mixed[r].push_back(std::make_shared<NDArrayView>(DataType::Float, 64, 4, 0));
        mixed[r].push_back(std::make_shared<NDArrayView>(DataType::Double, 64, 4, 0));
    }
    bool refused = false;
    try
    {
        two.QuantizedAggregateInPlace(mixed, res, stripe);
    }
    catch (const std::runtime_error& e)
    {
        refused = std::strstr(e.what(), "different types are not supported") != nullptr;
    }
    CHECK(refused, "a list of floats and doubles is refused");
    // residue lists of the wrong length
    PerWorker in = MakeValues<float>({{64, 4}, {64, 4}}, 2, 5), shortRes(2), s2(2);
    for (size_t r = 0; r < 2; ++r)
        shortRes[r].push_back(std::make_shared<NDArrayView>(DataType::Float, 64, 4, 0));
    bool logic = false;
    try
    {
        two.QuantizedAggregateInPlace(in, shortRes, s2);
    }
    catch (const std::logic_error&)
    {
        logic = true;
    }
    CHECK(logic, "a residue list of another length is a logic error");
    // one worker: nothing to aggregate, the inputs come back as outputs
    InProcessCommunicators one(1, false, true, 1);
    PerWorker single = MakeValues<float>({{64, 4}}, 1, 9), out(1), r1(1), s1(1), nr(1), ns(1);
    out[0].resize(1);
    one.QuantizedAggregate(single, r1, s1, out, nr, ns);
    CHECK(out[0].size() == 1 && out[0][0] == single[0][0], "single worker: output is the input");
    // no values: nothing happens
    PerWorker none(2), e1(2), e2(2);
    two.QuantizedAggregateInPlace(none, e1, e2);
    CHECK(e1[0].empty() && e2[1].empty(), "no values, no residues");
}

int main()
{
    try
    {
        struct T { const char* name; void (*fn)(); };
        const T tests[] = {{"OutOfPlaceEqualsAliasedFloat", OutOfPlaceFloat}, {"OutOfPlaceEqualsAliasedDouble", OutOfPlaceDouble},
                           {"EqualsAggregatorAndCallSequence", EqualsAggregatorAndCallSequence}, {"TypesAndTrivialCases", TypesAndTrivialCases}};
        for (const T& t : tests)
        {
            const int before = g_failures;
            t.fn();
            std::printf("Test case CommunicatorSuite/%s %s\n", t.name, g_failures != before ? "has FAILED" : "has passed");
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
