// Quantized all-reduce of gradient matrices: the reference's 1-bit-SGD aggregator restated over the MI355X quantizer,
// with the message transport factored out.
//
//   cntk_amd::AllReduceDistGradAggregator<float>  <->  Source/1BitSGD/AllReduceDistGradAggregator.h:20-631
//   cntk_amd::DistGradHeader                      <->  Source/SGDLib/DistGradHeader.h:5-100
//   cntk_amd::StripeTransport                          what the reference does with MPI point-to-point messages
//   cntk_amd::InProcessCluster                         K workers of one process sharing one GPU's memory
//
// Dataflow per worker r of K (Source/1BitSGD/AllReduceDistGradAggregator.h:237-566):
//   1. quantize every gradient with its carried residual                                   (:288-300)
//   2. hand stripe j of every packed gradient to worker j                                  (:303-378)
//   3. sum the K packed versions of the own stripe in fp32, requantize the sum with the
//      stripe residual, over the own slice of the own packed gradient                      (:365-375, 385-436)
//   4. hand the requantized stripe to every other worker                                   (:459-502)
//   5. unquantize the assembled packed gradient into the gradient matrix                   (:517-531)
//   The header (sample counts, criterion, evaluation errors) is summed on the main node and sent back (:380-383, 440-457).
//
// The reference runs one aggregator per MPI rank and interleaves the steps with blocking waits. Here the steps are three
// methods per worker (QuantizeAndPost, ReduceOwnStripes, FetchAndUnquantize) so that a single thread can drive K workers
// (InProcessCluster); a transport over real links would call the same methods around its own waits.
//
// Differences from the reference, all deliberate: packed gradients stay in device memory (the reference stages every
// stripe through pinned host memory); step 3 is one fused kernel when useFusedStripeReduce is set (bit-identical to the
// reference's sequence of calls, which remains available and is what useQuantizationForSelfStripe = false needs); the
// other workers' stripes are added in ascending rank order (the reference: message arrival order); the loops of steps 1
// and 5 can run as one launch each (useBatchedCalls).
#pragma once

#include "MatrixQuantizer.h"

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <deque>
#include <future>
#include <map>
#include <tuple>
#include <utility>

namespace cntk_amd {

// Source/SGDLib/DistGradHeader.h:5-100
struct DistGradHeader
{
    size_t numSamples = 0;
    size_t numSamplesWithLabel = 0; // denominator of 'criterion'
    double criterion = 0.0;
    std::vector<std::pair<double, size_t>> evalErrors; // (numerator, denominator) per evaluation node

    explicit DistGradHeader(int numEvalNode) : evalErrors((size_t) numEvalNode) {}
    int numEvalNode() const { return (int) evalErrors.size(); }

    void Aggregate(const DistGradHeader& other, bool add = false)
    {
        if (other.numEvalNode() != numEvalNode())
            throw std::runtime_error("mismatched size");
        if (!add)
        {
            *this = other;
            return;
        }
        numSamples += other.numSamples;
        numSamplesWithLabel += other.numSamplesWithLabel;
        criterion += other.criterion;
        for (size_t i = 0; i < evalErrors.size(); i++)
        {
            evalErrors[i].first += other.evalErrors[i].first;
            evalErrors[i].second += other.evalErrors[i].second;
        }
    }

    void Clear()
    {
        numSamples = numSamplesWithLabel = 0;
        criterion = 0;
        for (auto& e : evalErrors)
            e = {0.0, 0};
    }
};

// The messages of the quantized all-reduce. `from`, `to`, `owner` are worker ranks; a stripe is always the column range
// GetStripeForNode(cols, owner, K) of gradient matrix `matrixIdx`, as a packed matrix.
template <class ElemType>
class StripeTransportT
{
public:
    virtual ~StripeTransportT() {}
    virtual size_t NumProc() const = 0;
    // True when every message is device work on the quantizers' own stream, so that stream order alone keeps the steps
    // in sequence and the host waits the reference needs before handing buffers to MPI (:339, :494) can be skipped.
    virtual bool StreamOrdered() const { return false; }
    // Isend of a pre-aggregation stripe (Source/1BitSGD/AllReduceDistGradAggregator.h:339-365)
    virtual void PostStripe(size_t from, size_t to, size_t matrixIdx, QuantizedMatrix<ElemType>&& stripe) = 0;
    // what the matching Irecv delivered (:303-320)
    virtual const QuantizedMatrix<ElemType>& ReceivedStripe(size_t owner, size_t from, size_t matrixIdx) = 0;
    // Isend of the requantized stripe to everybody (:484-497) and its reception into the receiver's own packed gradient (:463-476)
    virtual void PostAggregatedStripe(size_t owner, size_t matrixIdx, QuantizedMatrix<ElemType>&& stripe) = 0;
    virtual void FetchAggregatedStripe(size_t to, size_t owner, size_t matrixIdx, QuantizedMatrix<ElemType>& dst, void* hipStream) = 0;
    // Where the receiver can read the owner's requantized stripe in place (same memory, or peer-accessible memory),
    // a view of it; nullptr where it has to be fetched into the receiver's own buffer first.
    virtual const QuantizedMatrix<ElemType>* AggregatedStripeView(size_t /*to*/, size_t /*owner*/, size_t /*matrixIdx*/) { return nullptr; }
    // headers to the main node and back (:323-333, 380-383, 440-457, 478-514)
    virtual void PostHeader(size_t from, const DistGradHeader& header) = 0;
    virtual DistGradHeader AggregatedHeader() = 0;
};

// All workers live in one process and their buffers in one GPU's memory: a stripe "message" is a view of the sender's
// buffer, the broadcast is a device-to-device copy on the quantizers' stream.
template <class ElemType>
class InProcessTransportT final : public StripeTransportT<ElemType>
{
public:
    explicit InProcessTransportT(size_t numWorkers, bool streamOrdered = true) : m_numWorkers(numWorkers), m_streamOrdered(streamOrdered) {}
    size_t NumProc() const override { return m_numWorkers; }
    bool StreamOrdered() const override { return m_streamOrdered; }

    void PostStripe(size_t from, size_t to, size_t matrixIdx, QuantizedMatrix<ElemType>&& stripe) override
    {
        Store(m_stripes, to * m_numWorkers + from, matrixIdx, std::move(stripe));
    }
    const QuantizedMatrix<ElemType>& ReceivedStripe(size_t owner, size_t from, size_t matrixIdx) override
    {
        const QuantizedMatrix<ElemType>* s = Find(m_stripes, owner * m_numWorkers + from, matrixIdx);
        if (s == nullptr)
            throw std::logic_error("InProcessTransport: stripe was never posted");
        return *s;
    }
    void PostAggregatedStripe(size_t owner, size_t matrixIdx, QuantizedMatrix<ElemType>&& stripe) override
    {
        Store(m_aggregated, owner, matrixIdx, std::move(stripe));
    }
    void FetchAggregatedStripe(size_t /*to*/, size_t owner, size_t matrixIdx, QuantizedMatrix<ElemType>& dst, void* hipStream) override
    {
        const QuantizedMatrix<ElemType>* s = Find(m_aggregated, owner, matrixIdx);
        if (s == nullptr)
            throw std::logic_error("InProcessTransport: aggregated stripe was never posted");
        if (s->GetSize() != dst.GetSize())
            throw std::logic_error("InProcessTransport: stripe size mismatch");
        if (dst.GetSize() != 0)
            detail::HipCheck(hipMemcpyAsync(dst.Buffer(), s->Buffer(), dst.GetSize(), hipMemcpyDeviceToDevice,
                                            static_cast<hipStream_t>(hipStream)),
                             "hipMemcpyAsync");
    }
    const QuantizedMatrix<ElemType>* AggregatedStripeView(size_t /*to*/, size_t owner, size_t matrixIdx) override
    {
        return Find(m_aggregated, owner, matrixIdx);
    }
    void PostHeader(size_t from, const DistGradHeader& header) override
    {
        m_headers.erase(from);
        m_headers.emplace(from, header);
    }
    DistGradHeader AggregatedHeader() override
    {
        // the main node starts from its own header and adds the others as they arrive (:440-457)
        if (m_headers.size() != m_numWorkers)
            throw std::logic_error("InProcessTransport: not every worker posted its header");
        DistGradHeader sum = m_headers.at(0);
        for (size_t r = 1; r < m_numWorkers; ++r)
            sum.Aggregate(m_headers.at(r), true);
        return sum;
    }

private:
    // messages by (channel, matrix); a message that names the very buffer of the previous step's is kept as it is,
    // so a steady training loop allocates nothing here
    typedef std::vector<std::vector<std::unique_ptr<QuantizedMatrix<ElemType>>>> Slots;
    static void Store(Slots& slots, size_t channel, size_t matrixIdx, QuantizedMatrix<ElemType>&& stripe)
    {
        if (slots.size() <= channel)
            slots.resize(channel + 1);
        if (slots[channel].size() <= matrixIdx)
            slots[channel].resize(matrixIdx + 1);
        std::unique_ptr<QuantizedMatrix<ElemType>>& slot = slots[channel][matrixIdx];
        if (slot && slot->Buffer() == stripe.Buffer() && slot->GetNumRows() == stripe.GetNumRows() &&
            slot->GetNumCols() == stripe.GetNumCols() && slot->GetNumBits() == stripe.GetNumBits())
            return;
        slot.reset(new QuantizedMatrix<ElemType>(std::move(stripe)));
    }
    static const QuantizedMatrix<ElemType>* Find(const Slots& slots, size_t channel, size_t matrixIdx)
    {
        if (channel >= slots.size() || matrixIdx >= slots[channel].size())
            return nullptr;
        return slots[channel][matrixIdx].get();
    }
    size_t m_numWorkers;
    bool m_streamOrdered;
    Slots m_stripes;
    Slots m_aggregated;
    std::map<size_t, DistGradHeader> m_headers;
};

// the float instantiation under the names of the message interface
typedef StripeTransportT<float> StripeTransport;
typedef InProcessTransportT<float> InProcessTransport;

template <class ElemType>
class AllReduceDistGradAggregator
{
public:
    struct Stripe
    {
        size_t m_startCol;
        size_t m_numCols;
    };

    struct Options
    {
        bool useFusedStripeReduce = true; // one kernel for "unquantize all stripes, sum, requantize"
        bool useBatchedCalls = true;      // one launch for all gradients in steps 1 and 5
        // InProcessCluster only: the K workers share one GPU and one stream, so the launches of all K workers in a step are
        // issued as ONE call each (K workers' quantize items in one grid; all K owners' stripes in one grid with an owner
        // per item; every worker's final unquantize in one grid). Same bytes as driving the workers one after another;
        // needs useFusedStripeReduce and useBatchedCalls, and falls back when a stripe is too tall for the fused call.
        bool useClusterBatching = true;
        // every syncStatsTrace-th aggregation is timed between two device synchronisations and reported on stderr as the
        // reference does ("Actual gradient aggregation time", Source/1BitSGD/AllReduceDistGradAggregator.h:153, 241-246,
        // 560-565); 0 = never
        int syncStatsTrace = 0;
        // from kDebugOutputTraceLevel on: the 3 x 3 corner of every gradient before it is quantized, of every packed stripe
        // that is sent, of every stripe that was received and of every aggregated gradient goes to stderr
        // (m_traceLevel >= DEBUG_OUTPUT_TRACE_LEVEL, Source/1BitSGD/AllReduceDistGradAggregator.h:37, 292-297, 351-361, 409-416,
        // 533-538); each peek waits for the device, so the steps no longer overlap
        int traceLevel = 0;
    };
    static const int kDebugOutputTraceLevel = 3;

    AllReduceDistGradAggregator(StripeTransportT<ElemType>& transport, size_t myRank, int deviceId, int nBits, bool zeroThresholdFor1Bit,
                                bool useQuantizationForSelfStripe, bool useAsyncAggregation, Options options = Options())
        : m_transport(transport), m_rank(myRank), m_deviceId(deviceId), m_numQuantizationBits((size_t) nBits),
          m_zeroThresholdFor1Bit(zeroThresholdFor1Bit), m_useQuantizationForSelfStripe(useQuantizationForSelfStripe),
          m_useAsyncAggregation(useAsyncAggregation), m_options(options), m_initialized(false)
    {
        if (myRank >= transport.NumProc())
            throw std::invalid_argument("AllReduceDistGradAggregator: rank out of range");
    }

    size_t MyRank() const { return m_rank; }
    size_t NumProc() const { return m_transport.NumProc(); }
    bool IsMainNode() const { return m_rank == 0; }

    // Source/1BitSGD/AllReduceDistGradAggregator.h:56-65
    static Stripe GetStripeForNode(size_t numCols, size_t nodeRank, size_t numNodes)
    {
        size_t start = 0, len = 0;
        detail::Check(cntkq_stripe_range(numCols, nodeRank, numNodes, &start, &len));
        return Stripe{start, len};
    }

    // First call: quantizers (with residuals) and packed buffers for every gradient and for the own stripe of every
    // gradient; later calls with resetState: all residuals back to zero (:67-147).
    void ResetState(const std::vector<Matrix<ElemType>*>& gradients, bool resetState)
    {
        if (!m_initialized)
        {
            m_initialized = true;
            for (size_t i = 0; i < gradients.size(); i++)
            {
                const size_t nRow = gradients[i]->GetNumRows(), nCol = gradients[i]->GetNumCols();
                m_preAggGradQuantizers.emplace_back(new MatrixQuantizer<ElemType>(nRow, nCol, m_deviceId, m_useAsyncAggregation));
                m_gradQuantized.emplace_back(new QuantizedMatrix<ElemType>(nRow, nCol, m_numQuantizationBits, m_deviceId));
                const Stripe stripe = GetStripeForNode(nCol, MyRank(), NumProc());
                MatrixQuantizer<ElemType>* stripeQuantizer = nullptr;
                if (stripe.m_numCols > 0)
                    stripeQuantizer = new MatrixQuantizer<ElemType>(nRow, stripe.m_numCols, m_deviceId, m_useAsyncAggregation);
                m_aggGradStripeQuantizers.emplace_back(stripeQuantizer);
            }
        }
        else if (resetState)
        {
            for (auto& q : m_preAggGradQuantizers)
                q->ResetResidue();
            for (auto& q : m_aggGradStripeQuantizers)
                if (q)
                    q->ResetResidue();
        }
        if (gradients.size() != m_preAggGradQuantizers.size())
            throw std::logic_error("AggregateGradients: the set of gradient matrices changed");
    }

    // Steps 1 and 2.
    void QuantizeAndPost(const std::vector<Matrix<ElemType>*>& gradients, DistGradHeader& headerCPU, bool resetState)
    {
        ResetState(gradients, resetState);
        const size_t numGradMatrices = gradients.size();
        // a worker that saw no samples contributes zero gradients (:250-266)
        if (headerCPU.numSamples == 0)
            for (auto* g : gradients)
                g->SetValue(0.0f);
        if (m_options.traceLevel >= kDebugOutputTraceLevel)
            for (size_t i = 0; i < numGradMatrices; ++i)
                PrintMatrix(Label("Original Gradient Matrix No. %d", i).c_str(), gradients[i]);
        // the gradients were produced on the main stream
        if (m_useAsyncAggregation && numGradMatrices > 0)
            SyncWithMainStream(*m_preAggGradQuantizers[0]);

        if (m_options.useBatchedCalls)
        {
            std::vector<typename MatrixQuantizerGPU<ElemType>::QuantizeItem> items;
            for (size_t i = 0; i < numGradMatrices; ++i)
                items.push_back({gradients[i], &m_preAggGradQuantizers[i]->GetResidualMatrix(), m_gradQuantized[i].get(),
                                 const_cast<Matrix<ElemType>*>(&m_preAggGradQuantizers[i]->GetResidualMatrix())});
            if (numGradMatrices > 0)
                Gpu(*m_preAggGradQuantizers[0]).QuantizeBatchAsync(items, m_zeroThresholdFor1Bit);
        }
        else
        {
            for (size_t i = 0; i < numGradMatrices; ++i)
                m_preAggGradQuantizers[i]->QuantizeAsync(*gradients[i], *m_gradQuantized[i], m_zeroThresholdFor1Bit);
        }

        const bool hostWaits = !m_transport.StreamOrdered();
        for (size_t i = 0; i < numGradMatrices; ++i)
        {
            if (hostWaits && !m_options.useBatchedCalls)
                m_preAggGradQuantizers[i]->WaitQuantizeAsyncDone(); // (:339)
            else if (hostWaits && i == 0)
                m_preAggGradQuantizers[0]->WaitQuantizeAsyncDone();
            for (size_t j = 0; j < NumProc(); ++j)
            {
                const Stripe stripe = GetStripeForNode(gradients[i]->GetNumCols(), j, NumProc());
                if (stripe.m_numCols == 0)
                    continue;
                // the owner's own stripe travels the same way: the fused reduction reads it like any other
                m_transport.PostStripe(MyRank(), j, i, m_gradQuantized[i]->ColumnSlice(stripe.m_startCol, stripe.m_numCols));
                if (m_options.traceLevel >= kDebugOutputTraceLevel && j != MyRank())
                    PeekQuantized(Label("Sending Gradient Matrix No. %d slice", i).c_str(),
                                  m_gradQuantized[i]->ColumnSlice(stripe.m_startCol, stripe.m_numCols));
            }
        }
        m_transport.PostHeader(MyRank(), headerCPU);
    }

    // Steps 3 and 4.
    void ReduceOwnStripes(const std::vector<Matrix<ElemType>*>& gradients)
    {
        const size_t K = NumProc();
        const bool fused = m_options.useFusedStripeReduce && m_useQuantizationForSelfStripe;
        // stripes that the fused call does not take keep the reference's sequence of calls
        auto fusable = [&](size_t i) {
            const size_t stripeCols = GetStripeForNode(gradients[i]->GetNumCols(), MyRank(), K).m_numCols;
            return fused && stripeCols != 0 &&
                   Gpu(*m_aggGradStripeQuantizers[i]).StripeReduceTakes(gradients[i]->GetNumRows(), stripeCols, m_numQuantizationBits, m_zeroThresholdFor1Bit);
        };
        if (m_options.traceLevel >= kDebugOutputTraceLevel)
            for (size_t i = 0; i < gradients.size(); ++i)
                for (size_t w = 0; w < K; ++w)
                    if (w != MyRank() && GetStripeForNode(gradients[i]->GetNumCols(), MyRank(), K).m_numCols != 0)
                        PeekQuantized(Label("Received Gradient Matrix No. %d slice", i).c_str(), m_transport.ReceivedStripe(MyRank(), w, i));
        // every matrix's stripe in one call: the stripe quantizers share one stream, so any of their handles will do
        const bool batched = fused && m_options.useBatchedCalls && gradients.size() > 1;
        if (batched)
        {
            typedef typename MatrixQuantizerGPU<ElemType>::StripeReduceItem Item;
            std::vector<Item> items;
            std::vector<QuantizedMatrix<ElemType>> ownSlices; // keep the views alive until the call
            ownSlices.reserve(gradients.size());
            for (size_t i = 0; i < gradients.size(); ++i)
            {
                const Stripe stripe = GetStripeForNode(gradients[i]->GetNumCols(), MyRank(), K);
                if (stripe.m_numCols == 0 || !fusable(i))
                    continue;
                ownSlices.push_back(m_gradQuantized[i]->ColumnSlice(stripe.m_startCol, stripe.m_numCols));
                Item it;
                for (size_t w = 0; w < K; ++w)
                    it.stripes.push_back(&m_transport.ReceivedStripe(MyRank(), w, i));
                it.stripeResidual = &const_cast<Matrix<ElemType>&>(m_aggGradStripeQuantizers[i]->GetResidualMatrix());
                it.outQStripe = &ownSlices.back();
                it.aggregate = nullptr;
                items.push_back(std::move(it));
            }
            if (!items.empty())
            {
                m_stripeBatchQuantizer = 0;
                while (GetStripeForNode(gradients[m_stripeBatchQuantizer]->GetNumCols(), MyRank(), K).m_numCols == 0 ||
                       !fusable(m_stripeBatchQuantizer))
                    m_stripeBatchQuantizer++;
                Gpu(*m_aggGradStripeQuantizers[m_stripeBatchQuantizer]).StripeReduceBatchAsync(items, MyRank(), m_zeroThresholdFor1Bit);
            }
        }
        for (size_t i = 0; i < gradients.size(); ++i)
        {
            const Stripe stripe = GetStripeForNode(gradients[i]->GetNumCols(), MyRank(), K);
            if (stripe.m_numCols == 0 || (batched && fusable(i)))
                continue;
            MatrixQuantizer<ElemType>& stripeQuantizer = *m_aggGradStripeQuantizers[i];
            QuantizedMatrix<ElemType> ownSlice = m_gradQuantized[i]->ColumnSlice(stripe.m_startCol, stripe.m_numCols);
            Matrix<ElemType>& stripeResidual = const_cast<Matrix<ElemType>&>(stripeQuantizer.GetResidualMatrix());
            if (fusable(i))
            {
                std::vector<const QuantizedMatrix<ElemType>*> stripes;
                for (size_t w = 0; w < K; ++w)
                    stripes.push_back(&m_transport.ReceivedStripe(MyRank(), w, i));
                Gpu(stripeQuantizer).StripeReduceAsync(stripes, MyRank(), stripeResidual, ownSlice, m_zeroThresholdFor1Bit);
            }
            else
            {
                // the reference's sequence: the aggregate lives in the own slice of the gradient matrix (:268-286)
                Matrix<ElemType> aggGradStripe = gradients[i]->ColumnSlice(stripe.m_startCol, stripe.m_numCols);
                if (m_useQuantizationForSelfStripe)
                    stripeQuantizer.UnquantizeAsync(ownSlice, aggGradStripe, false); // (:365-375)
                for (size_t w = 0; w < K; ++w)
                {
                    if (w == MyRank())
                        continue;
                    QuantizedMatrix<ElemType>& received = const_cast<QuantizedMatrix<ElemType>&>(m_transport.ReceivedStripe(MyRank(), w, i));
                    stripeQuantizer.UnquantizeAsync(received, aggGradStripe, true); // (:421)
                }
                // same stream: no wait needed between the last unquantize and the quantize (:426-434)
                stripeQuantizer.QuantizeAsync(aggGradStripe, ownSlice, m_zeroThresholdFor1Bit);
            }
        }
        const bool hostWaits = !m_transport.StreamOrdered();
        for (size_t i = 0; i < gradients.size(); ++i)
        {
            const Stripe stripe = GetStripeForNode(gradients[i]->GetNumCols(), MyRank(), K);
            if (stripe.m_numCols == 0)
                continue;
            if (hostWaits && batched && fusable(i))
                Gpu(*m_aggGradStripeQuantizers[m_stripeBatchQuantizer]).WaitStripeReduceDone();
            else if (hostWaits && fusable(i))
                Gpu(*m_aggGradStripeQuantizers[i]).WaitStripeReduceDone();
            else if (hostWaits)
                m_aggGradStripeQuantizers[i]->WaitQuantizeAsyncDone(); // (:494)
            m_transport.PostAggregatedStripe(MyRank(), i, m_gradQuantized[i]->ColumnSlice(stripe.m_startCol, stripe.m_numCols));
        }
    }

    // Step 5. Returns whether any worker processed samples (the reference's return value of AggregateGradients).
    bool FetchAndUnquantize(const std::vector<Matrix<ElemType>*>& gradients, DistGradHeader& headerCPU)
    {
        const size_t K = NumProc();
        // Stripes that can be read where their owner left them are unquantized straight from there, stripe by stripe;
        // the others are first gathered into the own packed gradient (:459-476), which is then unquantized whole (:517-522).
        std::vector<Matrix<ElemType>> outSlices;            // keep the views alive until the call below
        std::vector<QuantizedMatrix<ElemType>> ownSlices;
        std::vector<std::pair<const QuantizedMatrix<ElemType>*, size_t>> viewItems; // (packed stripe, index into outSlices)
        std::vector<bool> whole(gradients.size(), true);
        if (m_options.useBatchedCalls)
        {
            size_t slices = 0;
            for (size_t i = 0; i < gradients.size(); ++i)
                for (size_t j = 0; j < K; ++j)
                    slices += GetStripeForNode(gradients[i]->GetNumCols(), j, K).m_numCols > 0 ? 1 : 0;
            outSlices.reserve(slices);
            ownSlices.reserve(slices);
            for (size_t i = 0; i < gradients.size(); ++i)
            {
                bool allViews = true;
                for (size_t j = 0; j < K && allViews; ++j)
                    if (j != MyRank() && GetStripeForNode(gradients[i]->GetNumCols(), j, K).m_numCols > 0)
                        allViews = m_transport.AggregatedStripeView(MyRank(), j, i) != nullptr;
                if (!allViews)
                    continue;
                whole[i] = false;
                for (size_t j = 0; j < K; ++j)
                {
                    const Stripe stripe = GetStripeForNode(gradients[i]->GetNumCols(), j, K);
                    if (stripe.m_numCols == 0)
                        continue;
                    outSlices.push_back(gradients[i]->ColumnSlice(stripe.m_startCol, stripe.m_numCols));
                    if (j == MyRank())
                    {
                        ownSlices.push_back(m_gradQuantized[i]->ColumnSlice(stripe.m_startCol, stripe.m_numCols));
                        viewItems.push_back({&ownSlices.back(), outSlices.size() - 1});
                    }
                    else
                        viewItems.push_back({m_transport.AggregatedStripeView(MyRank(), j, i), outSlices.size() - 1});
                }
            }
        }
        for (size_t i = 0; i < gradients.size(); ++i)
        {
            if (!whole[i])
                continue;
            for (size_t j = 0; j < K; ++j)
            {
                if (j == MyRank())
                    continue;
                const Stripe stripe = GetStripeForNode(gradients[i]->GetNumCols(), j, K);
                if (stripe.m_numCols == 0)
                    continue;
                QuantizedMatrix<ElemType> dst = m_gradQuantized[i]->ColumnSlice(stripe.m_startCol, stripe.m_numCols);
                m_transport.FetchAggregatedStripe(MyRank(), j, i, dst, cntkq_stream(Gpu(*m_preAggGradQuantizers[i]).Handle()));
            }
        }
        if (m_options.useBatchedCalls)
        {
            std::vector<typename MatrixQuantizerGPU<ElemType>::UnquantizeItem> items;
            for (size_t i = 0; i < gradients.size(); ++i)
                if (whole[i])
                    items.push_back({m_gradQuantized[i].get(), gradients[i]});
            for (const auto& v : viewItems)
                items.push_back({v.first, &outSlices[v.second]});
            if (!items.empty())
            {
                Gpu(*m_preAggGradQuantizers[0]).UnquantizeBatchAsync(items, false);
                m_preAggGradQuantizers[0]->WaitUnquantizeAsyncDone();
            }
        }
        else
        {
            for (size_t i = 0; i < gradients.size(); ++i)
                m_preAggGradQuantizers[i]->UnquantizeAsync(*m_gradQuantized[i], *gradients[i], false); // (:521)
            for (size_t i = 0; i < gradients.size(); ++i)
                m_preAggGradQuantizers[i]->WaitUnquantizeAsyncDone();                                   // (:531)
        }
        if (m_options.traceLevel >= kDebugOutputTraceLevel)
            for (size_t i = 0; i < gradients.size(); ++i)
                PrintMatrix(Label("Aggregated Gradient Matrix No. %d", i).c_str(), gradients[i]);
        headerCPU.Aggregate(m_transport.AggregatedHeader(), false);
        return headerCPU.numSamples != 0;
    }

    // Debug helper: the 3 x 3 corner of a matrix (PrintMatrix with peek, Source/1BitSGD/AllReduceDistGradAggregator.h:568-587)
    static void PrintMatrix(const char* printHeader, const Matrix<ElemType>* matrixToPrint, FILE* out = stderr)
    {
        const size_t numRowsToPrint = (std::min)((size_t) 3, matrixToPrint->GetNumRows());
        const size_t numColsToPrint = (std::min)((size_t) 3, matrixToPrint->GetNumCols());
        if (numRowsToPrint != 0 && numColsToPrint != 0)
            matrixToPrint->Print(printHeader, 0, numRowsToPrint - 1, 0, numColsToPrint - 1, out);
        std::fflush(out);
    }
    // ... and of a packed matrix (:351-361)
    static void PeekQuantized(const char* printHeader, const QuantizedMatrix<ElemType>& q, FILE* out = stderr)
    {
        const size_t numRowsToPrint = (std::min)((size_t) 3, q.GetNumRows());
        const size_t numColsToPrint = (std::min)((size_t) 3, q.GetNumCols());
        if (numRowsToPrint != 0 && numColsToPrint != 0)
        {
            detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
            q.Print(printHeader, 0, numRowsToPrint - 1, 0, numColsToPrint - 1, out);
        }
        std::fflush(out);
    }
    std::string Label(const char* what, size_t matrixIdx) const
    {
        char buf[256];
        std::snprintf(buf, sizeof buf, (std::string("MPI Rank: %d, ") + what).c_str(), (int) MyRank(), (int) matrixIdx);
        return buf;
    }

    // ---- the same three steps cut into "which items" and "bookkeeping", for InProcessCluster's one call per step --------
    typedef MatrixQuantizerGPU<ElemType> GpuQuantizer;
    struct ClusterLaunch
    {
        std::vector<typename GpuQuantizer::QuantizeItem> quantize;
        std::vector<typename GpuQuantizer::StripeReduceItem> stripes;
        std::vector<size_t> owners;
        std::vector<typename GpuQuantizer::UnquantizeItem> unquantize;
        // views the items point to (deques: addresses stay valid while they grow)
        std::deque<QuantizedMatrix<ElemType>> packedViews;
        std::deque<Matrix<ElemType>> matrixViews;
    };

    // whether every own stripe of this gradient set can go through the fused call (then the cluster may batch)
    bool AllStripesFusable(const std::vector<Matrix<ElemType>*>& gradients) const
    {
        if (!(m_options.useFusedStripeReduce && m_useQuantizationForSelfStripe && m_options.useBatchedCalls && m_options.useClusterBatching))
            return false;
        if (m_options.traceLevel >= kDebugOutputTraceLevel)
            return false; // the debug peeks sit in the per-worker steps
        const size_t fusedMaxRows = detail::Abi<ElemType>::StripeReduceMaxRows(m_numQuantizationBits);
        for (auto* g : gradients)
            if (g->GetNumRows() > fusedMaxRows)
                return false;
        return m_transport.StreamOrdered();
    }

    // step 1 without the launch (:250-266, 288-300)
    void CollectQuantizeItems(const std::vector<Matrix<ElemType>*>& gradients, DistGradHeader& headerCPU, bool resetState, ClusterLaunch& launch)
    {
        ResetState(gradients, resetState);
        if (headerCPU.numSamples == 0)
            for (auto* g : gradients)
                g->SetValue(0.0f);
        for (size_t i = 0; i < gradients.size(); ++i)
            launch.quantize.push_back({gradients[i], &m_preAggGradQuantizers[i]->GetResidualMatrix(), m_gradQuantized[i].get(),
                                       const_cast<Matrix<ElemType>*>(&m_preAggGradQuantizers[i]->GetResidualMatrix())});
    }
    // step 2 on a stream-ordered transport
    void PostQuantized(const std::vector<Matrix<ElemType>*>& gradients, DistGradHeader& headerCPU)
    {
        for (size_t i = 0; i < gradients.size(); ++i)
            for (size_t j = 0; j < NumProc(); ++j)
            {
                const Stripe stripe = GetStripeForNode(gradients[i]->GetNumCols(), j, NumProc());
                if (stripe.m_numCols != 0)
                    m_transport.PostStripe(MyRank(), j, i, m_gradQuantized[i]->ColumnSlice(stripe.m_startCol, stripe.m_numCols));
            }
        m_transport.PostHeader(MyRank(), headerCPU);
    }
    // step 3 without the launch (:365-436): one item per gradient with an own stripe
    void CollectStripeItems(const std::vector<Matrix<ElemType>*>& gradients, ClusterLaunch& launch)
    {
        const size_t K = NumProc();
        for (size_t i = 0; i < gradients.size(); ++i)
        {
            const Stripe stripe = GetStripeForNode(gradients[i]->GetNumCols(), MyRank(), K);
            if (stripe.m_numCols == 0)
                continue;
            launch.packedViews.push_back(m_gradQuantized[i]->ColumnSlice(stripe.m_startCol, stripe.m_numCols));
            typename GpuQuantizer::StripeReduceItem it;
            for (size_t w = 0; w < K; ++w)
                it.stripes.push_back(&m_transport.ReceivedStripe(MyRank(), w, i));
            it.stripeResidual = &const_cast<Matrix<ElemType>&>(m_aggGradStripeQuantizers[i]->GetResidualMatrix());
            it.outQStripe = &launch.packedViews.back();
            it.aggregate = nullptr;
            launch.stripes.push_back(std::move(it));
            launch.owners.push_back(MyRank());
        }
    }
    // step 4 on a stream-ordered transport
    void PostReducedStripes(const std::vector<Matrix<ElemType>*>& gradients)
    {
        for (size_t i = 0; i < gradients.size(); ++i)
        {
            const Stripe stripe = GetStripeForNode(gradients[i]->GetNumCols(), MyRank(), NumProc());
            if (stripe.m_numCols != 0)
                m_transport.PostAggregatedStripe(MyRank(), i, m_gradQuantized[i]->ColumnSlice(stripe.m_startCol, stripe.m_numCols));
        }
    }
    // step 5 without the launch (:517-522): every stripe is decoded where its owner left it. False: some stripe cannot be
    // read in place (nothing was appended then, and the caller takes FetchAndUnquantize).
    bool CollectUnquantizeItems(const std::vector<Matrix<ElemType>*>& gradients, ClusterLaunch& launch)
    {
        const size_t K = NumProc();
        for (size_t i = 0; i < gradients.size(); ++i)
            for (size_t j = 0; j < K; ++j)
                if (j != MyRank() && GetStripeForNode(gradients[i]->GetNumCols(), j, K).m_numCols > 0 &&
                    m_transport.AggregatedStripeView(MyRank(), j, i) == nullptr)
                    return false;
        for (size_t i = 0; i < gradients.size(); ++i)
            for (size_t j = 0; j < K; ++j)
            {
                const Stripe stripe = GetStripeForNode(gradients[i]->GetNumCols(), j, K);
                if (stripe.m_numCols == 0)
                    continue;
                launch.matrixViews.push_back(gradients[i]->ColumnSlice(stripe.m_startCol, stripe.m_numCols));
                const QuantizedMatrix<ElemType>* packed = nullptr;
                if (j == MyRank())
                {
                    launch.packedViews.push_back(m_gradQuantized[i]->ColumnSlice(stripe.m_startCol, stripe.m_numCols));
                    packed = &launch.packedViews.back();
                }
                else
                    packed = m_transport.AggregatedStripeView(MyRank(), j, i);
                launch.unquantize.push_back({packed, &launch.matrixViews.back()});
            }
        return true;
    }
    bool FinishHeader(DistGradHeader& headerCPU)
    {
        headerCPU.Aggregate(m_transport.AggregatedHeader(), false);
        return headerCPU.numSamples != 0;
    }
    // the handles the cluster issues on (all quantizers of a cluster share one stream)
    GpuQuantizer* GradientQuantizerGpu() { return m_preAggGradQuantizers.empty() ? nullptr : &Gpu(*m_preAggGradQuantizers[0]); }
    GpuQuantizer* StripeQuantizerGpu()
    {
        for (auto& q : m_aggGradStripeQuantizers)
            if (q)
                return &Gpu(*q);
        return nullptr;
    }
    void SyncGradientQuantizerWithMainStream()
    {
        if (m_useAsyncAggregation && !m_preAggGradQuantizers.empty())
            SyncWithMainStream(*m_preAggGradQuantizers[0]);
    }
    bool ZeroThresholdFor1Bit() const { return m_zeroThresholdFor1Bit; }

    // Work this worker issues from now on starts only after `event` (a hipEvent_t recorded by the caller) has completed.
    // Needs the quantizers, i.e. a ResetState call before it.
    void WaitForEvent(void* event)
    {
        if (!m_preAggGradQuantizers.empty())
            detail::Check(cntkq_stream_wait_event(Gpu(*m_preAggGradQuantizers[0]).Handle(), event));
    }

    const Matrix<ElemType>& GradientResidual(size_t i) const { return m_preAggGradQuantizers[i]->GetResidualMatrix(); }
    const Matrix<ElemType>* StripeResidual(size_t i) const
    {
        return m_aggGradStripeQuantizers[i] ? &m_aggGradStripeQuantizers[i]->GetResidualMatrix() : nullptr;
    }
    const QuantizedMatrix<ElemType>& QuantizedGradient(size_t i) const { return *m_gradQuantized[i]; }

private:
    static MatrixQuantizerGPU<ElemType>& Gpu(MatrixQuantizer<ElemType>& q)
    {
        return dynamic_cast<MatrixQuantizerGPU<ElemType>&>(q.Impl());
    }
    void SyncWithMainStream(MatrixQuantizer<ElemType>& q)
    {
        std::unique_ptr<MatrixComputeStreamEvent> ev(MatrixComputeStreamEvent::Create(m_deviceId));
        ev->SynchronizeQuantizationComputeStreamWithEvent<ElemType>(q.Impl());
    }

    StripeTransportT<ElemType>& m_transport;
    size_t m_rank;
    int m_deviceId;
    size_t m_numQuantizationBits;
    bool m_zeroThresholdFor1Bit;
    bool m_useQuantizationForSelfStripe;
    bool m_useAsyncAggregation;
    Options m_options;
    bool m_initialized;

    std::vector<std::unique_ptr<MatrixQuantizer<ElemType>>> m_preAggGradQuantizers;
    std::vector<std::unique_ptr<QuantizedMatrix<ElemType>>> m_gradQuantized;
    std::vector<std::unique_ptr<MatrixQuantizer<ElemType>>> m_aggGradStripeQuantizers;
    size_t m_stripeBatchQuantizer = 0; // which of them carried the last batched stripe reduction
};

// K workers of one process on one GPU: drives the three steps of every worker in turn. This is the arrangement of the
// "K simulated workers in one GPU's memory" workload; a deployment has one worker per GPU and a transport over links.
template <class ElemType>
class InProcessCluster
{
public:
    typedef typename AllReduceDistGradAggregator<ElemType>::Options Options;

    // All quantizers of the cluster issue on one stream (the shared dedicated stream, or the main stream) and the transport is
    // stream-ordered: the K workers' steps are queued back to back and the host waits only at the very end.
    InProcessCluster(size_t numWorkers, int deviceId, int nBits, bool zeroThresholdFor1Bit, bool useQuantizationForSelfStripe = true,
                     bool useAsyncAggregation = true, Options options = Options())
        : m_transport(numWorkers, true), m_syncStatsTrace(options.syncStatsTrace)
    {
        for (size_t r = 0; r < numWorkers; ++r)
            m_workers.emplace_back(new AllReduceDistGradAggregator<ElemType>(m_transport, r, deviceId, nBits, zeroThresholdFor1Bit,
                                                                             useQuantizationForSelfStripe, useAsyncAggregation, options));
    }

    size_t NumWorkers() const { return m_workers.size(); }
    AllReduceDistGradAggregator<ElemType>& Worker(size_t r) { return *m_workers[r]; }

    // gradients[r] / headers[r] belong to worker r. With unquantizeOnAllWorkers = false only worker 0 ends up with the
    // aggregated gradients (the others would hold the same bytes); the packed aggregate is assembled on every worker.
    bool AggregateGradients(const std::vector<std::vector<Matrix<ElemType>*>>& gradients, std::vector<DistGradHeader>& headers,
                            bool resetState, bool unquantizeOnAllWorkers = true)
    {
        const size_t K = m_workers.size();
        if (gradients.size() != K || headers.size() != K)
            throw std::invalid_argument("InProcessCluster: one gradient set and one header per worker");
        const bool showSyncPerfStats = m_syncStatsTrace > 0 && (m_iterationCount % (size_t) m_syncStatsTrace) == 0;
        m_iterationCount++;
        std::chrono::steady_clock::time_point t0;
        if (showSyncPerfStats)
        {
            detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize"); // the gradients have been computed (:241-246)
            t0 = std::chrono::steady_clock::now();
        }
        bool clusterBatching = true;
        for (size_t r = 0; r < K; ++r)
            clusterBatching = clusterBatching && m_workers[r]->AllStripesFusable(gradients[r]);
        bool any = false;
        if (clusterBatching)
            any = AggregateAsOneCallPerStep(gradients, headers, resetState, unquantizeOnAllWorkers ? K : 1);
        else
        {
            for (size_t r = 0; r < K; ++r)
                m_workers[r]->QuantizeAndPost(gradients[r], headers[r], resetState);
            for (size_t r = 0; r < K; ++r)
                m_workers[r]->ReduceOwnStripes(gradients[r]);
            for (size_t r = 0; r < (unquantizeOnAllWorkers ? K : 1); ++r)
                any = m_workers[r]->FetchAndUnquantize(gradients[r], headers[r]) || any;
        }
        if (showSyncPerfStats)
        {
            detail::HipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
            const double seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
            std::fprintf(stderr, "Actual gradient aggregation time: %.6g\n", seconds);
        }
        return any;
    }

    // The K workers' steps with one call per step for the whole cluster (Options::useClusterBatching): the workers say which
    // matrices, stripes and views their step covers, and the cluster issues them together on the stream they all share.
    bool AggregateAsOneCallPerStep(const std::vector<std::vector<Matrix<ElemType>*>>& gradients, std::vector<DistGradHeader>& headers,
                                   bool resetState, size_t unquantizingWorkers)
    {
        const size_t K = m_workers.size();
        typename AllReduceDistGradAggregator<ElemType>::ClusterLaunch launch;
        for (size_t r = 0; r < K; ++r)
            m_workers[r]->CollectQuantizeItems(gradients[r], headers[r], resetState, launch);
        auto* gradientGpu = m_workers[0]->GradientQuantizerGpu();
        if (gradientGpu != nullptr)
        {
            m_workers[0]->SyncGradientQuantizerWithMainStream(); // the gradients were produced on the main stream
            gradientGpu->QuantizeBatchAsync(launch.quantize, m_workers[0]->ZeroThresholdFor1Bit());
        }
        for (size_t r = 0; r < K; ++r)
            m_workers[r]->PostQuantized(gradients[r], headers[r]);
        typename AllReduceDistGradAggregator<ElemType>::GpuQuantizer* stripeGpu = nullptr;
        for (size_t r = 0; r < K; ++r)
        {
            m_workers[r]->CollectStripeItems(gradients[r], launch);
            if (stripeGpu == nullptr)
                stripeGpu = m_workers[r]->StripeQuantizerGpu();
        }
        if (stripeGpu != nullptr && !launch.stripes.empty())
            stripeGpu->StripeReduceBatchAsync(launch.stripes, launch.owners, m_workers[0]->ZeroThresholdFor1Bit());
        for (size_t r = 0; r < K; ++r)
            m_workers[r]->PostReducedStripes(gradients[r]);
        bool any = false;
        std::vector<size_t> viaFetch;
        for (size_t r = 0; r < unquantizingWorkers; ++r)
            if (!m_workers[r]->CollectUnquantizeItems(gradients[r], launch))
                viaFetch.push_back(r);
        if (gradientGpu != nullptr && !launch.unquantize.empty())
        {
            gradientGpu->UnquantizeBatchAsync(launch.unquantize, false);
            gradientGpu->WaitUnquantizeAsyncDone();
        }
        for (size_t r = 0; r < unquantizingWorkers; ++r)
        {
            if (std::find(viaFetch.begin(), viaFetch.end(), r) != viaFetch.end())
                any = m_workers[r]->FetchAndUnquantize(gradients[r], headers[r]) || any;
            else
                any = m_workers[r]->FinishHeader(headers[r]) || any;
        }
        return any;
    }

    // The double-buffered aggregation of the reference (Source/1BitSGD/AllReduceDistGradAggregator.h:155-225, every
    // worker at once): waits for the aggregation started by the previous call, exchanges the contents of the gradient
    // matrices and headers with the buffered ones - the caller gets the gradients aggregated from the PREVIOUS call's
    // input (zeros the first time) - and starts aggregating what it was just given on another host thread, ordered after
    // everything already issued on the main (null) stream. As in the reference, aggregation starts only when state is
    // reset or the header coming back (the previous aggregate's) saw samples; the return value says whether it started.
    bool AggregateGradientsBuffered(const std::vector<std::vector<Matrix<ElemType>*>>& gradients, std::vector<DistGradHeader>& headers,
                                    bool resetState)
    {
        const size_t K = m_workers.size();
        if (gradients.size() != K || headers.size() != K)
            throw std::invalid_argument("InProcessCluster: one gradient set and one header per worker");
        WaitForPendingAggregation();
        if (m_buffered.empty())
        {
            m_buffered.resize(K);
            for (size_t r = 0; r < K; ++r)
            {
                for (auto* g : gradients[r])
                    m_buffered[r].emplace_back(new Matrix<ElemType>(g->GetNumRows(), g->GetNumCols(), g->GetDeviceId()));
                m_bufferedHeaders.emplace_back(headers[r].numEvalNode());
            }
        }
        std::vector<std::vector<Matrix<ElemType>*>> fresh(K);
        for (size_t r = 0; r < K; ++r)
        {
            if (gradients[r].size() != m_buffered[r].size())
                throw std::logic_error("No buffered gradient matrix found corresponding to a gradient matrix to be aggregated!");
            for (size_t i = 0; i < gradients[r].size(); ++i)
            {
                Matrix<ElemType>& b = *m_buffered[r][i];
                if (b.GetNumRows() != gradients[r][i]->GetNumRows() || b.GetNumCols() != gradients[r][i]->GetNumCols() ||
                    b.GetDeviceId() != gradients[r][i]->GetDeviceId())
                    throw std::logic_error("No buffered gradient matrix found corresponding to a gradient matrix to be aggregated!");
                gradients[r][i]->Swap(b);
                fresh[r].push_back(&b);
            }
            std::swap(headers[r], m_bufferedHeaders[r]);
        }
        if (!(resetState || headers[0].numSamples != 0))
            return false;
        int device = 0;
        detail::HipCheck(hipGetDevice(&device), "hipGetDevice");
        hipEvent_t computed = nullptr;
        detail::HipCheck(hipEventCreateWithFlags(&computed, hipEventDisableTiming), "hipEventCreate");
        detail::HipCheck(hipEventRecord(computed, nullptr), "hipEventRecord");
        for (size_t r = 0; r < K; ++r)
            m_workers[r]->ResetState(fresh[r], false); // the quantizers exist before the other thread needs their stream
        m_pending = std::async(std::launch::async, [this, fresh, device, computed, resetState]() {
            detail::HipCheck(hipSetDevice(device), "hipSetDevice");
            m_workers[0]->WaitForEvent(computed);
            AggregateGradients(fresh, m_bufferedHeaders, resetState, true);
            detail::HipCheck(hipEventDestroy(computed), "hipEventDestroy");
        });
        return true;
    }

    void WaitForPendingAggregation()
    {
        if (m_pending.valid())
            m_pending.get();
    }

    ~InProcessCluster()
    {
        try
        {
            WaitForPendingAggregation();
        }
        catch (...)
        {
        }
    }

private:
    InProcessTransportT<ElemType> m_transport;
    std::vector<std::unique_ptr<AllReduceDistGradAggregator<ElemType>>> m_workers;
    std::vector<std::vector<std::unique_ptr<Matrix<ElemType>>>> m_buffered;
    std::vector<DistGradHeader> m_bufferedHeaders;
    std::future<void> m_pending;
    int m_syncStatsTrace = 0;
    size_t m_iterationCount = 0;
};

} // namespace cntk_amd
