// Tests of the quantized data-parallel learner mirror (cntk_amd/cpp/QuantizedDataParallelDistributedLearner.h) with K
// ranks in one process on one GPU. What the reference's learner tests assert for this class
// (bindings/python/cntk/learners/tests/distributed_learner_test.py:101-158): local training until distributeAfterSamples
// samples have been seen, then every rank updates with the same aggregated gradients and sample count; plus the pieces of
// Update the reference implements around the aggregation (Source/1BitSGD/QuantizedDataParallelDistributedLearner.h:29-97):
// zero gradients from a rank with an empty minibatch, no update when all ranks are empty, residuals cleared by a checkpoint,
// gradients paired across ranks by parameter Uid.
#include "../../cntk_amd/cpp/QuantizedDataParallelDistributedLearner.h"

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

static std::vector<float> Gaussian(size_t n, float sigma, unsigned long seed)
{
    std::mt19937_64 rng(seed);
    std::normal_distribution<float> d(0.0f, sigma);
    std::vector<float> a(n);
    for (auto& x : a)
        x = d(rng);
    return a;
}

static std::vector<float> Host(const Matrix<float>& m)
{
    auto a = m.CopyToArray();
    return std::vector<float>(a.get(), a.get() + m.GetNumElements());
}

// Plain SGD on host copies of the parameters: w -= lr * g / samples. Records what it was called with.
class SgdLearner final : public Learner<float>
{
public:
    explicit SgdLearner(const std::vector<std::pair<std::string, size_t>>& params)
    {
        for (const auto& p : params)
            weights[p.first] = std::vector<float>(p.second, 1.0f);
    }
    bool Update(GradientValues& gradientValues, size_t trainingSampleCount, bool) override
    {
        calls++;
        lastSampleCount = trainingSampleCount;
        for (auto& g : gradientValues)
        {
            const std::vector<float> h = Host(*g.second);
            std::vector<float>& w = weights.at(g.first);
            for (size_t i = 0; i < w.size(); ++i)
                w[i] -= 0.1f * h[i] / (float) trainingSampleCount;
        }
        return true;
    }
    std::unordered_map<std::string, std::vector<float>> weights;
    int calls = 0;
    size_t lastSampleCount = 0;
};

struct Param
{
    std::string uid;
    size_t rows, cols;
};

struct Rank
{
    std::vector<std::unique_ptr<Matrix<float>>> owned;
    Learner<float>::GradientValues grads;
};

// rank r inserts its parameters in an order of its own: the pairing across ranks must come from the Uids
static std::vector<Rank> MakeRanks(const std::vector<Param>& params, size_t K, const std::vector<std::vector<std::vector<float>>>& host)
{
    std::vector<Rank> ranks(K);
    for (size_t r = 0; r < K; ++r)
        for (size_t n = 0; n < params.size(); ++n)
        {
            const size_t i = (n * 2 + r) % params.size(); // a permutation: params.size() is odd
            ranks[r].owned.emplace_back(new Matrix<float>(params[i].rows, params[i].cols, 0));
            ranks[r].owned.back()->SetValue(host[r][i].data());
            ranks[r].grads[params[i].uid] = ranks[r].owned.back().get();
        }
    return ranks;
}

static std::vector<std::vector<std::vector<float>>> MakeHost(const std::vector<Param>& params, size_t K, unsigned long seed)
{
    std::vector<std::vector<std::vector<float>>> host(K);
    for (size_t r = 0; r < K; ++r)
        for (size_t i = 0; i < params.size(); ++i)
            host[r].push_back(Gaussian(params[i].rows * params[i].cols, 0.01f, seed + 100 * r + i));
    return host;
}

static const std::vector<Param> kParams = {{"Parameter7", 64, 24}, {"Parameter12", 64, 24}, {"Parameter3", 64, 24}, {"Parameter40", 128, 9},
                                           {"Parameter5", 33, 7}};

// Uid order (plain string order, as the reference sorts)
static std::vector<size_t> UidOrder()
{
    std::vector<size_t> idx(kParams.size());
    for (size_t i = 0; i < idx.size(); ++i)
        idx[i] = i;
    std::sort(idx.begin(), idx.end(), [](size_t a, size_t b) { return kParams[a].uid < kParams[b].uid; });
    return idx;
}

static void WarmStartThenExactSum()
{
    const size_t K = 4, perRank = 32, distributeAfter = 64;
    std::vector<std::pair<std::string, size_t>> sizes;
    for (const auto& p : kParams)
        sizes.push_back({p.uid, p.rows * p.cols});
    InProcessCluster<float> cluster(K, 0, 32, false); // 32 bits: the aggregate is the plain fp32 sum in rank order from the owner
    std::vector<std::unique_ptr<SgdLearner>> sgd;
    std::vector<Learner<float>*> learners;
    for (size_t r = 0; r < K; ++r)
    {
        sgd.emplace_back(new SgdLearner(sizes));
        learners.push_back(sgd.back().get());
    }
    InProcessLearnerGroup<float> group(cluster, learners, distributeAfter);
    for (int step = 0; step < 4; ++step)
    {
        const auto host = MakeHost(kParams, K, 777 + 1000 * step);
        std::vector<Rank> ranks = MakeRanks(kParams, K, host);
        std::vector<Learner<float>::GradientValues> grads;
        std::vector<MinibatchInfo> infos(K);
        for (size_t r = 0; r < K; ++r)
        {
            grads.push_back(ranks[r].grads);
            infos[r].numberOfSamples = perRank;
            infos[r].trainingLossValue = 2.0 + r;
            infos[r].evalCriterionValue = 0.5 * r;
        }
        const bool distributing = group.Rank(0).Distributing();
        CHECK(distributing == (step >= 2), "aggregation starts once %zu samples were seen (step %d)", distributeAfter, step);
        const std::vector<bool> updated = group.Update(grads, infos);
        detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
        for (size_t r = 0; r < K; ++r)
        {
            CHECK(updated[r] && sgd[r]->calls == step + 1, "rank %zu updated", r);
            if (!distributing)
            {
                // local training: own gradients untouched, own sample count
                CHECK(infos[r].numberOfSamples == perRank && sgd[r]->lastSampleCount == perRank, "local sample count");
                for (size_t i = 0; i < kParams.size(); ++i)
                    CHECK(Host(*grads[r].at(kParams[i].uid)) == host[r][i], "warm start leaves gradients alone (rank %zu, %s)", r,
                          kParams[i].uid.c_str());
                CHECK(group.Rank(r).TotalNumberOfSamplesSeen() == (size_t) (step + 1) * perRank, "samples seen, local phase");
            }
            else
            {
                CHECK(infos[r].numberOfSamples == K * perRank && sgd[r]->lastSampleCount == K * perRank, "aggregated sample count");
                CHECK(std::fabs(infos[r].trainingLossValue - (2.0 * K + 6.0)) < 1e-12 && std::fabs(infos[r].evalCriterionValue - 3.0) < 1e-12,
                      "loss and criterion are summed");
                CHECK(group.Rank(r).TotalNumberOfSamplesSeen() == 2 * perRank + (size_t) (step - 1) * K * perRank, "samples seen, distributed phase");
                for (size_t i = 0; i < kParams.size(); ++i)
                {
                    // parameter i on every rank: the sum over ranks of THAT parameter's gradients
                    const std::vector<float> got = Host(*grads[r].at(kParams[i].uid));
                    const size_t rows = kParams[i].rows, cols = kParams[i].cols;
                    bool ok = true;
                    for (size_t c = 0; c < cols && ok; ++c)
                    {
                        // the column's owner sums its own contribution first, then the others in ascending rank order
                        size_t owner = 0;
                        for (size_t s = 0; s < K; ++s)
                        {
                            size_t start, len;
                            cntkq_stripe_range(cols, s, K, &start, &len);
                            if (c >= start && c < start + len)
                                owner = s;
                        }
                        for (size_t x = 0; x < rows && ok; ++x)
                        {
                            float sum = host[owner][i][c * rows + x];
                            for (size_t s = 0; s < K; ++s)
                                if (s != owner)
                                    sum = host[s][i][c * rows + x] + sum;
                            ok = std::memcmp(&sum, &got[c * rows + x], 4) == 0;
                        }
                    }
                    CHECK(ok, "rank %zu, %s: aggregated gradient is the sum of this parameter's gradients", r, kParams[i].uid.c_str());
                }
            }
        }
    }
    std::printf("DistributedLearnerWarmStartThenExactSum has passed\n");
}

static void OneBitMatchesTheAggregatorInUidOrder()
{
    const size_t K = 4;
    std::vector<std::pair<std::string, size_t>> sizes;
    for (const auto& p : kParams)
        sizes.push_back({p.uid, p.rows * p.cols});
    const std::vector<size_t> order = UidOrder();
    InProcessCluster<float> clusterA(K, 0, 1, false), clusterB(K, 0, 1, false);
    std::vector<std::unique_ptr<SgdLearner>> sgd;
    std::vector<Learner<float>*> learners;
    for (size_t r = 0; r < K; ++r)
    {
        sgd.emplace_back(new SgdLearner(sizes));
        learners.push_back(sgd.back().get());
    }
    InProcessLearnerGroup<float> group(clusterA, learners, 0);
    bool checkpointed = false;
    std::unique_ptr<InProcessCluster<float>> fresh;
    for (int step = 0; step < 5; ++step)
    {
        const auto host = MakeHost(kParams, K, 31 + 1000 * step);
        std::vector<Rank> ranks = MakeRanks(kParams, K, host);
        std::vector<Learner<float>::GradientValues> grads;
        std::vector<MinibatchInfo> infos(K);
        // step 1: rank 2 has no data (and whatever is in its gradient buffers must not count); step 3: nobody has data
        for (size_t r = 0; r < K; ++r)
        {
            grads.push_back(ranks[r].grads);
            infos[r].numberOfSamples = (step == 3 || (step == 1 && r == 2)) ? 0 : 16;
        }
        // the same step on the aggregator directly, gradients in Uid order
        std::vector<Rank> direct = MakeRanks(kParams, K, host);
        std::vector<std::vector<Matrix<float>*>> ordered(K);
        std::vector<DistGradHeader> headers;
        for (size_t r = 0; r < K; ++r)
        {
            for (size_t i : order)
                ordered[r].push_back(direct[r].grads.at(kParams[i].uid));
            headers.emplace_back(1);
            headers.back().numSamples = infos[r].numberOfSamples;
        }
        InProcessCluster<float>& expect = checkpointed ? *fresh : clusterB;
        const int callsBefore = sgd[0]->calls;
        const std::vector<bool> updated = group.Update(grads, infos);
        expect.AggregateGradients(ordered, headers, false, true);
        detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
        for (size_t r = 0; r < K; ++r)
        {
            CHECK(updated[r] == (step != 3), "step %d rank %zu: update happens unless every rank is empty", step, r);
            CHECK(infos[r].numberOfSamples == headers[r].numSamples, "aggregated sample count");
            for (const auto& p : kParams)
                CHECK(Host(*grads[r].at(p.uid)) == Host(*direct[r].grads.at(p.uid)), "step %d rank %zu %s: same bytes as the aggregator in Uid order",
                      step, r, p.uid.c_str());
        }
        CHECK(sgd[0]->calls == callsBefore + (step != 3 ? 1 : 0), "local learner skipped when all ranks are empty");
        if (step == 1)
            CHECK(sgd[2]->lastSampleCount == 48, "the empty rank still updates, with the others' samples");
        if (step == 2)
        {
            // checkpoint: residuals are cleared, so the following steps equal those of a cluster that starts now
            const std::vector<size_t> state = group.CreateCheckpoint();
            CHECK(state.size() == K && state[0] == group.Rank(0).TotalNumberOfSamplesSeen() && state[0] == 64 + 48 + 64, "checkpoint holds the samples seen");
            fresh.reset(new InProcessCluster<float>(K, 0, 1, false));
            checkpointed = true;
        }
    }
    for (size_t r = 0; r < K; ++r)
        for (size_t i = 0; i < kParams.size(); ++i)
            CHECK(Host(clusterA.Worker(r).GradientResidual(i)) == Host(fresh->Worker(r).GradientResidual(i)), "residuals after a checkpoint (rank %zu, gradient %zu)", r, i);
    // restore: sample count back, residuals cleared again
    group.Rank(0).RestoreFromCheckpoint(123);
    CHECK(group.Rank(0).TotalNumberOfSamplesSeen() == 123, "restore");
    bool thrown = false;
    try
    {
        QuantizedDataParallelDistributedLearner<float> bad(clusterA.Worker(0), *learners[0], 0, true);
    }
    catch (const std::logic_error&)
    {
        thrown = true;
    }
    CHECK(thrown, "asynchronous buffered updates are refused");
    std::printf("DistributedLearnerOneBitUidOrderEmptyAndCheckpoint has passed\n");
}

int main()
{
    try
    {
        WarmStartThenExactSum();
        OneBitMatchesTheAggregatorInUidOrder();
    }
    catch (const std::exception& e)
    {
        std::fprintf(stderr, "exception: %s\n", e.what());
        return 2;
    }
    if (g_failures)
    {
        std::fprintf(stderr, "%d checks failed\n", g_failures);
        return 1;
    }
    std::printf("all distributed learner tests passed\n");
    return 0;
}
