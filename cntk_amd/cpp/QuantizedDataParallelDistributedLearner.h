// Host-side mirror of the reference's quantized data-parallel learner
// (Source/1BitSGD/QuantizedDataParallelDistributedLearner.h:29-118, Source/CNTKv2LibraryDll/DistributedLearnerBase.cpp:15-118)
// over the quantized all-reduce aggregator of this library: which gradients go into the aggregation, in which order, when
// aggregation starts, what happens on an empty minibatch, what a checkpoint does to the residuals.
//
// The reference's Update is one blocking collective per rank. Here its two exchange points are explicit
// (BeginUpdate / ReduceStripes / FinishUpdate), so that the K ranks of one process on one GPU can be driven in turn by
// InProcessLearnerGroup; a deployment with one rank per GPU calls the three in sequence.
#pragma once

#include "AllReduceDistGradAggregator.h"

#include <string>
#include <unordered_map>

namespace cntk_amd {

// bindings' MinibatchInfo (Source/CNTKv2LibraryDll/API/CNTKLibrary.h: MinibatchInfo)
struct MinibatchInfo
{
    bool atEndOfData = false;
    bool atEndOfSweep = false;
    size_t numberOfSamples = 0;
    double trainingLossValue = 0.0;
    double evalCriterionValue = 0.0;
    bool IsEmpty() const { return numberOfSamples == 0; }
};

// The local learner a distributed learner wraps: applies (aggregated) gradients to the parameters it owns.
template <class ElemType>
class Learner
{
public:
    typedef std::unordered_map<std::string, Matrix<ElemType>*> GradientValues; // parameter Uid -> gradient
    virtual ~Learner() {}
    virtual bool Update(GradientValues& gradientValues, size_t trainingSampleCount, bool sweepEnd) = 0;
};

template <class ElemType>
class QuantizedDataParallelDistributedLearner
{
public:
    typedef typename Learner<ElemType>::GradientValues GradientValues;

    // distributeAfterSamples: until the learner has seen that many samples it trains locally, without aggregation
    // (the warm start of DistributedLearnerBase). Asynchronous buffered updates are refused like in the reference (:24-25).
    QuantizedDataParallelDistributedLearner(AllReduceDistGradAggregator<ElemType>& communicator, Learner<ElemType>& learner,
                                            size_t distributeAfterSamples, bool useAsyncBufferedParameterUpdate = false)
        : m_communicator(communicator), m_learner(learner), m_distributeAfterSamples(distributeAfterSamples), m_sampleCount(0),
          m_header(1), m_resetResiduals(false), m_aggregating(false)
    {
        if (useAsyncBufferedParameterUpdate)
            throw std::logic_error("Asynchronous parameter update is not yet supported.");
    }

    size_t TotalNumberOfSamplesSeen() const { return m_sampleCount; }
    bool Distributing() const { return m_sampleCount >= m_distributeAfterSamples; }

    // First third of Update (:31-62): zero gradients for an empty minibatch, gradients ordered by parameter Uid so that
    // gradient i (and residual i) is the same parameter on every rank, header (criterion, loss, sample count) and packed
    // gradients posted.
    void BeginUpdate(GradientValues& gradientValues, const MinibatchInfo& info)
    {
        m_aggregating = Distributing();
        if (!m_aggregating)
            return;
        ConvertToOrdered(gradientValues);
        m_header.Clear();
        m_header.numSamples = info.numberOfSamples;
        m_header.numSamplesWithLabel = info.numberOfSamples;
        m_header.criterion = info.trainingLossValue;
        m_header.evalErrors[0] = {info.evalCriterionValue, info.numberOfSamples};
        // (a rank without samples contributes zero gradients: the aggregator clears them when the header says so)
        m_communicator.QuantizeAndPost(m_ordered, m_header, m_resetResiduals);
        m_resetResiduals = false;
    }

    // The stripes this rank owns: decode, sum, requantize with the stripe residual.
    void ReduceStripes()
    {
        if (m_aggregating)
            m_communicator.ReduceOwnStripes(m_ordered);
    }

    // Last third (:47-76): aggregated header and gradients back, the sample count advanced by the AGGREGATED number of
    // samples, then the local learner, unless no rank had data.
    bool FinishUpdate(GradientValues& gradientValues, MinibatchInfo& info)
    {
        if (m_aggregating)
        {
            m_communicator.FetchAndUnquantize(m_ordered, m_header);
            info.numberOfSamples = m_header.numSamples;
            info.trainingLossValue = m_header.criterion;
            info.evalCriterionValue = m_header.evalErrors[0].first;
            m_ordered.clear();
        }
        m_sampleCount += info.numberOfSamples;
        if (info.IsEmpty())
            return false;
        return m_learner.Update(gradientValues, info.numberOfSamples, info.atEndOfSweep);
    }

    // One rank per process: the whole collective.
    bool Update(GradientValues& gradientValues, MinibatchInfo& info)
    {
        BeginUpdate(gradientValues, info);
        ReduceStripes();
        return FinishUpdate(gradientValues, info);
    }

    // The residuals are not part of a checkpoint, so taking one clears them: the state in memory then equals the state a
    // restore produces (:80-97). Returns what the base class stores: the number of samples seen (DistributedLearnerBase.cpp:78-90).
    size_t CreateCheckpoint()
    {
        m_resetResiduals = true; // applied by the aggregator before the next quantization
        return m_sampleCount;
    }

    void RestoreFromCheckpoint(size_t totalNumberOfSamplesSeen)
    {
        m_sampleCount = totalNumberOfSamplesSeen;
        m_resetResiduals = true;
    }

private:
    // DistributedLearnerBase::ConvertToOrdered (DistributedLearnerBase.cpp:49-76)
    void ConvertToOrdered(const GradientValues& gradientValues)
    {
        std::vector<std::pair<std::string, Matrix<ElemType>*>> sorted(gradientValues.begin(), gradientValues.end());
        std::sort(sorted.begin(), sorted.end(), [](const auto& a, const auto& b) { return a.first < b.first; });
        m_ordered.clear();
        for (const auto& p : sorted)
            m_ordered.push_back(p.second);
    }

    AllReduceDistGradAggregator<ElemType>& m_communicator;
    Learner<ElemType>& m_learner;
    size_t m_distributeAfterSamples;
    size_t m_sampleCount;
    DistGradHeader m_header;
    std::vector<Matrix<ElemType>*> m_ordered;
    bool m_resetResiduals;
    bool m_aggregating;
};

// The K ranks of one process: every rank's BeginUpdate, then every rank's ReduceStripes, then every rank's FinishUpdate.
template <class ElemType>
class InProcessLearnerGroup
{
public:
    typedef typename Learner<ElemType>::GradientValues GradientValues;

    InProcessLearnerGroup(InProcessCluster<ElemType>& cluster, const std::vector<Learner<ElemType>*>& learners, size_t distributeAfterSamples)
    {
        if (learners.size() != cluster.NumWorkers())
            throw std::invalid_argument("InProcessLearnerGroup: one local learner per worker");
        for (size_t r = 0; r < learners.size(); ++r)
            m_ranks.emplace_back(new QuantizedDataParallelDistributedLearner<ElemType>(cluster.Worker(r), *learners[r], distributeAfterSamples));
    }

    QuantizedDataParallelDistributedLearner<ElemType>& Rank(size_t r) { return *m_ranks[r]; }

    // returns, per rank, what that rank's Update returned
    std::vector<bool> Update(std::vector<GradientValues>& gradientValues, std::vector<MinibatchInfo>& infos)
    {
        if (gradientValues.size() != m_ranks.size() || infos.size() != m_ranks.size())
            throw std::invalid_argument("InProcessLearnerGroup: one gradient set and one MinibatchInfo per worker");
        for (size_t r = 0; r < m_ranks.size(); ++r)
            m_ranks[r]->BeginUpdate(gradientValues[r], infos[r]);
        for (size_t r = 0; r < m_ranks.size(); ++r)
            m_ranks[r]->ReduceStripes();
        std::vector<bool> updated(m_ranks.size());
        for (size_t r = 0; r < m_ranks.size(); ++r)
            updated[r] = m_ranks[r]->FinishUpdate(gradientValues[r], infos[r]);
        return updated;
    }

    std::vector<size_t> CreateCheckpoint()
    {
        std::vector<size_t> state;
        for (auto& r : m_ranks)
            state.push_back(r->CreateCheckpoint());
        return state;
    }

private:
    std::vector<std::unique_ptr<QuantizedDataParallelDistributedLearner<ElemType>>> m_ranks;
};

} // namespace cntk_amd
