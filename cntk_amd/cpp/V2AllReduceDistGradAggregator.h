// The reference's gradient aggregator over the v2 communicator, restated over the MI355X quantizer.
//
//   cntk_amd::V2AllReduceDistGradAggregator  <->  V2AllReduceDistGradAggregator (Source/1BitSGD/V2AllReduceDistGradAggregator.h:30-297)
//
// What this aggregator is, next to the v1 one (AllReduceDistGradAggregator.h): it owns no quantizer and no packed buffer.
// It keeps two lists of residues that start empty and are filled by the communicator's first call (:285-295), sends the
// header as a vector of doubles through the communicator's plain aggregation (:228-253: criterion, numSamples,
// numSamplesWithLabel, then numerator and denominator of every evaluation node) and the gradients, wrapped as views of
// the caller's matrices (:256-263), through QuantizedAggregateInPlace (:265-269). A worker that saw no samples sends
// zeros as gradients (:213-226). With useAsyncAggregation the caller's gradients and header are exchanged with buffered
// ones on every call, and what was handed in is aggregated while the caller computes the next gradients (:114-186).
//
// One process drives K workers on one GPU here, so the collective calls of the K workers happen together: a worker's
// object (V2AllReduceDistGradAggregator) holds the state of one rank and the parts of a call that concern that rank
// alone; InProcessV2Aggregators makes the K workers' calls, with the two collective steps in the middle.
#pragma once

#include "QuantizedDistributedCommunicator.h"

#include <future>
#include <unordered_map>

namespace cntk_amd {

// One rank's state and the rank-local parts of AggregateGradients.
template <class ElemType>
class V2AllReduceDistGradAggregator
{
public:
    // (:39-43; the communicator belongs to InProcessV2Aggregators here)
    V2AllReduceDistGradAggregator(bool useAsyncAggregation, int traceLevel, int syncStatsTrace)
        : m_useAsyncAggregation(useAsyncAggregation), m_bufferedGradHeader(0), m_traceLevel(traceLevel), m_syncStatsTrace(syncStatsTrace),
          m_iterationCount(0), m_initialized(false)
    {
    }

    // (:51-75)
    void Initialize(const std::vector<Matrix<ElemType>*>& gradients, int numEvalNodes)
    {
        m_initialized = true;
        if (gradients.empty())
            throw std::invalid_argument("V2AllReduceDistGradAggregator: no gradients");
        const int deviceId = gradients[0]->GetDeviceId();
        if (m_useAsyncAggregation)
        {
            for (auto* g : gradients)
                m_bufferedGradients[g].reset(new Matrix<ElemType>(g->GetNumRows(), g->GetNumCols(), deviceId));
            m_bufferedGradHeader = DistGradHeader(numEvalNodes);
            m_bufferedGradHeader.Clear();
        }
    }

    // (:77-97) `pending`: an aggregation started by an earlier call has not been waited for
    void ResetState(const std::vector<Matrix<ElemType>*>& gradients, bool pending)
    {
        if (m_useAsyncAggregation && pending)
            throw std::logic_error("Unexpected pending async gradient aggregation found when resetting aggregator state!");
        for (auto& r : m_residuals)
            r->template GetWritableMatrix<ElemType>()->SetValue((ElemType) 0);
        for (auto& r : m_stripeResiduals)
            if (r)
                r->template GetWritableMatrix<ElemType>()->SetValue((ElemType) 0);
        if (m_useAsyncAggregation)
        {
            for (auto* g : gradients)
                BufferedFor(g).SetValue((ElemType) 0);
            m_bufferedGradHeader.Clear();
        }
    }

    // (:103-107) what AggregateGradients does before anything else
    void InitializeOrReset(const std::vector<Matrix<ElemType>*>& gradients, const DistGradHeader& headerCPU, bool resetState, bool pending)
    {
        if (!m_initialized)
            Initialize(gradients, headerCPU.numEvalNode());
        else if (resetState)
            ResetState(gradients, pending);
    }

    // (:109-110)
    bool NextCallShowsStats()
    {
        const bool show = m_syncStatsTrace > 0 && (m_iterationCount % (size_t) m_syncStatsTrace) == 0;
        m_iterationCount++;
        return show;
    }

    // (:131-154) the caller's gradients and header change places with the buffered ones; returns the matrices that now
    // hold what the caller handed in, and leaves that call's header in BufferedHeader()
    std::vector<Matrix<ElemType>*> SwapWithBuffered(const std::vector<Matrix<ElemType>*>& gradients, DistGradHeader& headerCPU)
    {
        std::vector<Matrix<ElemType>*> newGradients;
        for (auto* g : gradients)
        {
            Matrix<ElemType>& b = BufferedFor(g);
            g->Swap(b);
            newGradients.push_back(&b);
        }
        std::swap(headerCPU, m_bufferedGradHeader);
        return newGradients;
    }
    DistGradHeader& BufferedHeader() { return m_bufferedGradHeader; }

    // (:213-226) a worker without samples contributes zeros
    void ZeroGradientsIfNoSamples(const std::vector<Matrix<ElemType>*>& gradients, const DistGradHeader& headerCPU)
    {
        if (headerCPU.numSamples != 0)
            return;
        for (auto* g : gradients)
            g->SetValue((ElemType) 0);
    }

    // (:228-239)
    static std::vector<double> PackHeader(const DistGradHeader& h)
    {
        std::vector<double> buffer(3 + 2 * h.evalErrors.size());
        buffer[0] = h.criterion;
        buffer[1] = (double) h.numSamples;
        buffer[2] = (double) h.numSamplesWithLabel;
        for (size_t i = 0; i < h.evalErrors.size(); ++i)
        {
            buffer[3 + 2 * i] = h.evalErrors[i].first;
            buffer[3 + 2 * i + 1] = (double) h.evalErrors[i].second;
        }
        return buffer;
    }

    // (:246-253)
    static void UnpackHeader(const std::vector<double>& buffer, DistGradHeader& h)
    {
        if (buffer.size() != 3 + 2 * h.evalErrors.size())
            throw std::logic_error("V2AllReduceDistGradAggregator: header of another size");
        h.criterion = buffer[0];
        h.numSamples = (size_t) buffer[1];
        h.numSamplesWithLabel = (size_t) buffer[2];
        for (size_t i = 0; i < h.evalErrors.size(); ++i)
        {
            h.evalErrors[i].first = buffer[3 + 2 * i];
            h.evalErrors[i].second = (size_t) buffer[3 + 2 * i + 1];
        }
    }

    // (:256-263) the gradients as values of the communicator: views of the caller's memory
    static std::vector<NDArrayViewPtr> GradientValues(const std::vector<Matrix<ElemType>*>& gradients)
    {
        std::vector<NDArrayViewPtr> values;
        for (auto* g : gradients)
        {
            if (g->Data() == nullptr)
                throw std::logic_error("V2AllReduceDistGradAggregator: a gradient without memory");
            values.push_back(std::make_shared<NDArrayView>(std::make_shared<Matrix<ElemType>>(g->ColumnSlice(0, g->GetNumCols()))));
        }
        return values;
    }

    bool UseAsyncAggregation() const { return m_useAsyncAggregation; }
    int TraceLevel() const { return m_traceLevel; }
    std::vector<NDArrayViewPtr>& Residuals() { return m_residuals; }
    std::vector<NDArrayViewPtr>& StripeResiduals() { return m_stripeResiduals; }

private:
    Matrix<ElemType>& BufferedFor(Matrix<ElemType>* g)
    {
        auto it = m_bufferedGradients.find(g);
        Matrix<ElemType>* b = it == m_bufferedGradients.end() ? nullptr : it->second.get();
        if (b == nullptr || b->GetNumCols() != g->GetNumCols() || b->GetNumRows() != g->GetNumRows() || b->GetDeviceId() != g->GetDeviceId())
            throw std::logic_error("No buffered gradient matrix found corresponding to a gradient matrix to be aggregated!");
        return *b;
    }

    bool m_useAsyncAggregation;
    std::unordered_map<Matrix<ElemType>*, std::unique_ptr<Matrix<ElemType>>> m_bufferedGradients; // (:275)
    DistGradHeader m_bufferedGradHeader;
    int m_traceLevel;
    int m_syncStatsTrace;
    size_t m_iterationCount;
    bool m_initialized;
    std::vector<NDArrayViewPtr> m_residuals;       // residues of the quantized gradients (:292)
    std::vector<NDArrayViewPtr> m_stripeResiduals; // residues of the stripes this worker aggregates (:294)
};

// The K workers' aggregators of one process on one GPU, over K communicators of the same process.
template <class ElemType>
class InProcessV2Aggregators
{
public:
    InProcessV2Aggregators(size_t numWorkers, bool zeroThresholdFor1Bit, bool useQuantizationForSelfStripe, size_t numQuantizationBits,
                           bool useAsyncAggregation, int traceLevel = 0, int syncStatsTrace = 0,
                           QuantizedCommunicator::Options options = QuantizedCommunicator::Options())
        : m_communicators(numWorkers, zeroThresholdFor1Bit, useQuantizationForSelfStripe, numQuantizationBits, options)
    {
        for (size_t r = 0; r < numWorkers; ++r)
            m_workers.emplace_back(new V2AllReduceDistGradAggregator<ElemType>(useAsyncAggregation, traceLevel, syncStatsTrace));
    }
    ~InProcessV2Aggregators()
    {
        try
        {
            WaitForPendingAggregation();
        }
        catch (...)
        {
        }
    }

    size_t NumWorkers() const { return m_workers.size(); }
    V2AllReduceDistGradAggregator<ElemType>& Worker(size_t r) { return *m_workers[r]; }

    // AggregateGradients of every worker at once (:100-188): gradients[r] and headers[r] are worker r's arguments, the
    // return value is worker 0's (the aggregated header is the same on every worker, and so is resetState).
    bool AggregateGradients(const std::vector<std::vector<Matrix<ElemType>*>>& gradients, std::vector<DistGradHeader>& headers, bool resetState)
    {
        const size_t K = m_workers.size();
        if (gradients.size() != K || headers.size() != K)
            throw std::invalid_argument("InProcessV2Aggregators: one gradient set and one header per worker");
        const bool pending = m_pending.valid();
        for (size_t r = 0; r < K; ++r)
            m_workers[r]->InitializeOrReset(gradients[r], headers[r], resetState, pending);
        bool showSyncPerfStats = false;
        for (size_t r = 0; r < K; ++r)
            showSyncPerfStats = m_workers[r]->NextCallShowsStats() || showSyncPerfStats;

        if (!m_workers[0]->UseAsyncAggregation())
        {
            AggregateGradientsImpl(gradients, headers, showSyncPerfStats);
            return headers[0].numSamples != 0;
        }

        if (m_pending.valid())
        {
            const auto t0 = std::chrono::steady_clock::now();
            m_pending.get();
            if (showSyncPerfStats)
                std::fprintf(stderr, "Async gradient aggregation wait time: %.6g\n",
                             std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count());
        }
        std::vector<std::vector<Matrix<ElemType>*>> newGradients(K);
        for (size_t r = 0; r < K; ++r)
            newGradients[r] = m_workers[r]->SwapWithBuffered(gradients[r], headers[r]);
        // aggregation starts only if the previous one saw samples anywhere, or on a reset (:157)
        if (!(resetState || headers[0].numSamples != 0))
            return false;
        // the gradients have been computed on the main stream by the time the other thread starts on them (:162-178)
        int device = 0;
        detail::HipCheck(hipGetDevice(&device), "hipGetDevice");
        hipEvent_t computed = nullptr;
        detail::HipCheck(hipEventCreateWithFlags(&computed, hipEventDisableTiming), "hipEventCreate");
        detail::HipCheck(hipEventRecord(computed, nullptr), "hipEventRecord");
        m_pending = std::async(std::launch::async, [this, newGradients, device, computed, showSyncPerfStats]() {
            detail::HipCheck(hipSetDevice(device), "hipSetDevice");
            detail::HipCheck(hipEventSynchronize(computed), "hipEventSynchronize");
            detail::HipCheck(hipEventDestroy(computed), "hipEventDestroy");
            std::vector<DistGradHeader*> bufferedHeaders;
            for (auto& w : m_workers)
                bufferedHeaders.push_back(&w->BufferedHeader());
            AggregateGradientsImpl(newGradients, bufferedHeaders, showSyncPerfStats);
        });
        return true;
    }

    void WaitForPendingAggregation()
    {
        if (m_pending.valid())
            m_pending.get();
    }

private:
    void AggregateGradientsImpl(const std::vector<std::vector<Matrix<ElemType>*>>& gradients, std::vector<DistGradHeader>& headers,
                                bool showSyncPerfStats)
    {
        std::vector<DistGradHeader*> pointers;
        for (auto& h : headers)
            pointers.push_back(&h);
        AggregateGradientsImpl(gradients, pointers, showSyncPerfStats);
    }

    // (:190-283), every worker at once
    void AggregateGradientsImpl(const std::vector<std::vector<Matrix<ElemType>*>>& gradients, const std::vector<DistGradHeader*>& headers,
                                bool showSyncPerfStats)
    {
        const size_t K = m_workers.size();
        std::chrono::steady_clock::time_point t0;
        if (showSyncPerfStats)
        {
            detail::HipCheck(hipStreamSynchronize(nullptr), "hipStreamSynchronize");
            t0 = std::chrono::steady_clock::now();
        }
        for (size_t r = 0; r < K; ++r)
            m_workers[r]->ZeroGradientsIfNoSamples(gradients[r], *headers[r]);

        // the header, as doubles through the plain aggregation
        std::vector<std::vector<double>> packed(K);
        for (size_t r = 0; r < K; ++r)
            packed[r] = V2AllReduceDistGradAggregator<ElemType>::PackHeader(*headers[r]);
        m_communicators.AggregateInPlace(packed);
        for (size_t r = 0; r < K; ++r)
            V2AllReduceDistGradAggregator<ElemType>::UnpackHeader(packed[r], *headers[r]);

        // the gradients, through the quantized aggregation, with this aggregator's residues
        InProcessCommunicators::PerWorker values(K), residuals(K), stripeResiduals(K);
        for (size_t r = 0; r < K; ++r)
        {
            values[r] = V2AllReduceDistGradAggregator<ElemType>::GradientValues(gradients[r]);
            residuals[r] = m_workers[r]->Residuals();
            stripeResiduals[r] = m_workers[r]->StripeResiduals();
        }
        m_communicators.QuantizedAggregateInPlace(values, residuals, stripeResiduals);
        for (size_t r = 0; r < K; ++r)
        {
            m_workers[r]->Residuals() = residuals[r];
            m_workers[r]->StripeResiduals() = stripeResiduals[r];
        }
        if (showSyncPerfStats)
        {
            detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
            std::fprintf(stderr, "Actual gradient aggregation time: %.6g\n",
                         std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count());
        }
    }

    InProcessCommunicators m_communicators;
    std::vector<std::unique_ptr<V2AllReduceDistGradAggregator<ElemType>>> m_workers;
    std::future<void> m_pending;
};

} // namespace cntk_amd
