// The v2 communicator's quantized aggregation restated over the MI355X quantizer, with the message transport factored out.
//
//   cntk_amd::QuantizedCommunicator  <->  CNTK::QuantizedMPICommunicatorImpl (Source/1BitSGD/QuantizedDistributedCommunicator.h:27-566)
//   cntk_amd::NDArrayView            <->  what the communicator uses of CNTK::NDArrayView: element type, shape, device, the matrix
//
// What differs from the v1 aggregator (AllReduceDistGradAggregator.h) is the call shape, and that is what this file keeps:
//   * values and residues are the caller's (NDArrayView lists), not members: QuantizedAggregate takes inValues,
//     valueQuantizationResidues, stripeQuantizationResidues and writes aggregatedOutputs, newQuantizationResidues,
//     newStripeQuantizationResidues, which may be other buffers or the same ones (QuantizedAggregateInPlace, :51-62);
//   * empty residue lists are filled with freshly allocated zero residues on the first call, two buffers per gradient
//     (an input and an output one) as InitializeBuffer does (:236-251);
//   * float or double is taken from the values on every call; a list that mixes them is refused (:84-90), sparse values do
//     not exist here;
//   * a communicator of one worker hands the inputs back as outputs (:72-78);
//   * the quantizers own no residual (MatrixQuantizer(deviceId, useAsync), :258-266), and the fp32 aggregate of the own
//     stripe is accumulated in the own stripe of the INPUT value, as the reference does (:347-353).
// The dataflow (:364-539) is the aggregator's: quantize every value with its residue -> stripe j of every packed value to
// worker j -> own stripe: unquantize own (if useQuantizationForSelfStripe), add the others, requantize with the stripe
// residue over the own slice of the packed value -> requantized stripes to everyone -> unquantize the assembled packed
// value into the output. As in AllReduceDistGradAggregator.h it is cut into three methods per worker around a
// StripeTransport, so that one thread can drive K workers of one process (InProcessCommunicators below); packed values
// stay in device memory; the other workers' stripes are added in ascending rank order where the reference adds them as
// they arrive.
// Stripe reduction: with useFusedStripeReduce the one fused call (which updates a stripe residue in place: distinct
// input and output residues are served by copying the input over the output first, on the same stream); without it the
// reference's sequence of calls. Both give the same bytes.
#pragma once

#include "AllReduceDistGradAggregator.h"

#include <memory>
#include <string>

namespace cntk_amd {

enum class DataType
{
    Float,
    Double
};

// The part of CNTK::NDArrayView this path touches: a dense column-major matrix of floats or doubles on one device.
class NDArrayView
{
public:
    NDArrayView(DataType type, size_t numRows, size_t numCols, int deviceId) : m_type(type)
    {
        if (type == DataType::Float)
            m_float = std::make_shared<Matrix<float>>(numRows, numCols, deviceId);
        else
            m_double = std::make_shared<Matrix<double>>(numRows, numCols, deviceId);
    }
    // over a matrix that exists (possibly a view of the caller's memory)
    explicit NDArrayView(std::shared_ptr<Matrix<float>> m) : m_type(DataType::Float), m_float(std::move(m)) {}
    explicit NDArrayView(std::shared_ptr<Matrix<double>> m) : m_type(DataType::Double), m_double(std::move(m)) {}
    DataType GetDataType() const { return m_type; }
    size_t GetNumRows() const { return m_float ? m_float->GetNumRows() : m_double->GetNumRows(); }
    size_t GetNumCols() const { return m_float ? m_float->GetNumCols() : m_double->GetNumCols(); }
    int GetDeviceId() const { return m_float ? m_float->GetDeviceId() : m_double->GetDeviceId(); }

    template <class ElemType>
    std::shared_ptr<Matrix<ElemType>> GetWritableMatrix() const;

private:
    DataType m_type;
    std::shared_ptr<Matrix<float>> m_float;
    std::shared_ptr<Matrix<double>> m_double;
};
template <>
inline std::shared_ptr<Matrix<float>> NDArrayView::GetWritableMatrix<float>() const
{
    if (!m_float)
        throw std::logic_error("Unexpected type value.");
    return m_float;
}
template <>
inline std::shared_ptr<Matrix<double>> NDArrayView::GetWritableMatrix<double>() const
{
    if (!m_double)
        throw std::logic_error("Unexpected type value.");
    return m_double;
}
typedef std::shared_ptr<NDArrayView> NDArrayViewPtr;

template <class ElemType>
inline DataType AsDataType();
template <>
inline DataType AsDataType<float>() { return DataType::Float; }
template <>
inline DataType AsDataType<double>() { return DataType::Double; }

struct QuantizedCommunicatorOptions
{
    bool useFusedStripeReduce = true; // one kernel for "unquantize all stripes, sum, requantize"
};

class QuantizedCommunicator
{
public:
    typedef QuantizedCommunicatorOptions Options;

    // One transport per element type: a call uses the one of its values' type.
    QuantizedCommunicator(StripeTransportT<float>& floatTransport, StripeTransportT<double>& doubleTransport, size_t myRank,
                          bool zeroThresholdFor1Bit, bool useQuantizationForSelfStripe, size_t numQuantizationBits, Options options = Options())
        : m_floatTransport(floatTransport), m_doubleTransport(doubleTransport), m_rank(myRank), m_zeroThresholdFor1Bit(zeroThresholdFor1Bit),
          m_useQuantizationForSelfStripe(useQuantizationForSelfStripe), m_numQuantizationBits(numQuantizationBits), m_options(options)
    {
        if (floatTransport.NumProc() != doubleTransport.NumProc() || myRank >= floatTransport.NumProc())
            throw std::invalid_argument("QuantizedCommunicator: transports of equal size and a rank below it");
    }

    size_t NumWorkers() const { return m_floatTransport.NumProc(); }
    size_t Rank() const { return m_rank; }

    // What a call works on; filled by Begin, used by the three steps. The lists the caller passed are completed in place
    // (missing residues allocated), as the reference completes its by-value copies and output arguments.
    struct Call
    {
        DataType dataType = DataType::Float;
        bool trivial = false; // one worker, or nothing to aggregate
        std::vector<NDArrayViewPtr> inValues, valueResidues, stripeResidues, outputs, newValueResidues, newStripeResidues;
    };

    // The argument handling of QuantizedAggregate up to the typed call (:64-96, 179-233).
    Call Begin(const std::vector<NDArrayViewPtr>& inValues, std::vector<NDArrayViewPtr>& valueQuantizationResidues,
               std::vector<NDArrayViewPtr>& stripeQuantizationResidues, std::vector<NDArrayViewPtr>& aggregatedOutputs,
               std::vector<NDArrayViewPtr>& newQuantizationResidues, std::vector<NDArrayViewPtr>& newStripeQuantizationResidues)
    {
        Call call;
        if (NumWorkers() == 1) // no need to aggregate anything
        {
            aggregatedOutputs = inValues;
            newQuantizationResidues = valueQuantizationResidues;
            newStripeQuantizationResidues = stripeQuantizationResidues;
            call.trivial = true;
            return call;
        }
        if (inValues.empty())
        {
            call.trivial = true;
            return call;
        }
        call.dataType = inValues.front()->GetDataType();
        for (const auto& v : inValues)
            if (v->GetDataType() != call.dataType)
                throw std::runtime_error("Currently values of different types are not supported for quantize.");
        if (std::max(inValues.size(), valueQuantizationResidues.size()) != inValues.size())
            throw std::logic_error("Number of aggregated values should be equal number of quantized residuals.");
        if (std::max(inValues.size(), stripeQuantizationResidues.size()) != inValues.size())
            throw std::logic_error("Number of aggregated values should be equal number of striped quantized residuals.");
        if (aggregatedOutputs.size() != inValues.size())
            throw std::logic_error("Number of aggregated values should be equal number of outputs.");
        if (valueQuantizationResidues.empty())
            valueQuantizationResidues.resize(inValues.size());
        if (stripeQuantizationResidues.empty())
            stripeQuantizationResidues.resize(inValues.size());
        if (newQuantizationResidues.empty())
            newQuantizationResidues.resize(inValues.size());
        if (newStripeQuantizationResidues.empty())
            newStripeQuantizationResidues.resize(inValues.size());
        if (valueQuantizationResidues.size() != inValues.size() || stripeQuantizationResidues.size() != inValues.size() ||
            newQuantizationResidues.size() != inValues.size() || newStripeQuantizationResidues.size() != inValues.size())
            throw std::logic_error("Number of aggregated values should be equal number of quantized residuals.");
        for (size_t i = 0; i < inValues.size(); ++i)
        {
            const size_t nRow = inValues[i]->GetNumRows(), nCol = inValues[i]->GetNumCols();
            const int device = inValues[i]->GetDeviceId();
            if (!valueQuantizationResidues[i])
            {
                valueQuantizationResidues[i] = std::make_shared<NDArrayView>(call.dataType, nRow, nCol, device);
                newQuantizationResidues[i] = std::make_shared<NDArrayView>(call.dataType, nRow, nCol, device);
            }
            const auto stripe = AllReduceDistGradAggregator<float>::GetStripeForNode(nCol, m_rank, NumWorkers());
            if (!stripeQuantizationResidues[i] && stripe.m_numCols > 0)
            {
                stripeQuantizationResidues[i] = std::make_shared<NDArrayView>(call.dataType, nRow, stripe.m_numCols, device);
                newStripeQuantizationResidues[i] = std::make_shared<NDArrayView>(call.dataType, nRow, stripe.m_numCols, device);
            }
            if (!aggregatedOutputs[i] || !newQuantizationResidues[i] || (stripe.m_numCols > 0 && !newStripeQuantizationResidues[i]))
                throw std::logic_error("QuantizedAggregate: an output buffer is missing");
            if (aggregatedOutputs[i]->GetNumRows() != nRow || aggregatedOutputs[i]->GetNumCols() != nCol ||
                aggregatedOutputs[i]->GetDataType() != call.dataType)
                throw std::logic_error("QuantizedAggregate: output does not match its input");
        }
        call.inValues = inValues;
        call.valueResidues = valueQuantizationResidues;
        call.stripeResidues = stripeQuantizationResidues;
        call.outputs = aggregatedOutputs;
        call.newValueResidues = newQuantizationResidues;
        call.newStripeResidues = newStripeQuantizationResidues;
        return call;
    }

    // the three steps, dispatched on the element type of the call
    void QuantizeAndPost(Call& call)
    {
        if (call.trivial)
            return;
        call.dataType == DataType::Float ? QuantizeAndPostT<float>(call, m_floatTransport, m_float) : QuantizeAndPostT<double>(call, m_doubleTransport, m_double);
    }
    void ReduceOwnStripes(Call& call)
    {
        if (call.trivial)
            return;
        call.dataType == DataType::Float ? ReduceOwnStripesT<float>(call, m_floatTransport, m_float) : ReduceOwnStripesT<double>(call, m_doubleTransport, m_double);
    }
    void FetchAndUnquantize(Call& call)
    {
        if (call.trivial)
            return;
        call.dataType == DataType::Float ? FetchAndUnquantizeT<float>(call, m_floatTransport, m_float) : FetchAndUnquantizeT<double>(call, m_doubleTransport, m_double);
    }

private:
    template <class ElemType>
    struct State // InitializeBuffer's members (:553-565), per element type
    {
        std::vector<std::unique_ptr<MatrixQuantizer<ElemType>>> preAggregatedGradientQuantizers;
        std::vector<std::unique_ptr<QuantizedMatrix<ElemType>>> quantizedGradients;
        std::vector<std::unique_ptr<MatrixQuantizer<ElemType>>> aggregatedGradientStripeQuantizers;
    };

    template <class ElemType>
    static MatrixQuantizerGPU<ElemType>& Gpu(MatrixQuantizer<ElemType>& q)
    {
        return dynamic_cast<MatrixQuantizerGPU<ElemType>&>(q.Impl());
    }

    // (re)creates quantizers and packed buffers when the list of shapes changes (the reference rebuilds them on every call)
    template <class ElemType>
    void InitializeBuffers(const Call& call, State<ElemType>& st)
    {
        bool same = st.quantizedGradients.size() == call.inValues.size();
        for (size_t i = 0; same && i < call.inValues.size(); ++i)
            same = st.quantizedGradients[i]->GetNumRows() == call.inValues[i]->GetNumRows() &&
                   st.quantizedGradients[i]->GetNumCols() == call.inValues[i]->GetNumCols();
        if (same)
            return;
        st = State<ElemType>();
        for (size_t i = 0; i < call.inValues.size(); ++i)
        {
            const size_t nRow = call.inValues[i]->GetNumRows(), nCol = call.inValues[i]->GetNumCols();
            const int device = call.inValues[i]->GetDeviceId();
            st.quantizedGradients.emplace_back(new QuantizedMatrix<ElemType>(nRow, nCol, m_numQuantizationBits, device));
            st.preAggregatedGradientQuantizers.emplace_back(new MatrixQuantizer<ElemType>(device, true));
            const auto stripe = AllReduceDistGradAggregator<ElemType>::GetStripeForNode(nCol, m_rank, NumWorkers());
            st.aggregatedGradientStripeQuantizers.emplace_back(stripe.m_numCols > 0 ? new MatrixQuantizer<ElemType>(device, true) : nullptr);
        }
    }

    template <class ElemType>
    void QuantizeAndPostT(Call& call, StripeTransportT<ElemType>& transport, State<ElemType>& st)
    {
        InitializeBuffers(call, st);
        const size_t K = NumWorkers();
        // the values were produced on the main stream
        if (!call.inValues.empty())
        {
            std::unique_ptr<MatrixComputeStreamEvent> ev(MatrixComputeStreamEvent::Create(call.inValues[0]->GetDeviceId()));
            ev->SynchronizeQuantizationComputeStreamWithEvent<ElemType>(st.preAggregatedGradientQuantizers[0]->Impl());
        }
        for (size_t i = 0; i < call.inValues.size(); ++i) // (:364-366)
            st.preAggregatedGradientQuantizers[i]->QuantizeAsync(*call.inValues[i]->template GetWritableMatrix<ElemType>(),
                                                                 *call.valueResidues[i]->template GetWritableMatrix<ElemType>(), *st.quantizedGradients[i],
                                                                 *call.newValueResidues[i]->template GetWritableMatrix<ElemType>(), m_zeroThresholdFor1Bit);
        const bool hostWaits = !transport.StreamOrdered();
        for (size_t i = 0; i < call.inValues.size(); ++i)
        {
            if (hostWaits)
                st.preAggregatedGradientQuantizers[i]->WaitQuantizeAsyncDone(); // (:393)
            for (size_t j = 0; j < K; ++j)
            {
                const auto stripe = AllReduceDistGradAggregator<ElemType>::GetStripeForNode(call.inValues[i]->GetNumCols(), j, K);
                if (stripe.m_numCols > 0)
                    transport.PostStripe(m_rank, j, i, st.quantizedGradients[i]->ColumnSlice(stripe.m_startCol, stripe.m_numCols));
            }
        }
    }

    template <class ElemType>
    void ReduceOwnStripesT(Call& call, StripeTransportT<ElemType>& transport, State<ElemType>& st)
    {
        const size_t K = NumWorkers();
        for (size_t i = 0; i < call.inValues.size(); ++i)
        {
            const auto stripe = AllReduceDistGradAggregator<ElemType>::GetStripeForNode(call.inValues[i]->GetNumCols(), m_rank, K);
            if (stripe.m_numCols == 0)
                continue;
            MatrixQuantizer<ElemType>& stripeQuantizer = *st.aggregatedGradientStripeQuantizers[i];
            QuantizedMatrix<ElemType> ownSlice = st.quantizedGradients[i]->ColumnSlice(stripe.m_startCol, stripe.m_numCols);
            Matrix<ElemType>& inStripeResidue = *call.stripeResidues[i]->template GetWritableMatrix<ElemType>();
            Matrix<ElemType>& outStripeResidue = *call.newStripeResidues[i]->template GetWritableMatrix<ElemType>();
            const bool fused = m_options.useFusedStripeReduce && m_useQuantizationForSelfStripe &&
                               Gpu(stripeQuantizer).StripeReduceTakes(call.inValues[i]->GetNumRows(), stripe.m_numCols, m_numQuantizationBits,
                                                                      m_zeroThresholdFor1Bit);
            if (fused)
            {
                // the fused call updates one residue in place: distinct buffers get the input's contents first
                if (outStripeResidue.Data() != inStripeResidue.Data())
                    detail::HipCheck(hipMemcpyAsync(outStripeResidue.Data(), inStripeResidue.Data(), inStripeResidue.GetNumElements() * sizeof(ElemType),
                                                    hipMemcpyDeviceToDevice, static_cast<hipStream_t>(cntkq_stream(Gpu(stripeQuantizer).Handle()))),
                                     "hipMemcpyAsync");
                std::vector<const QuantizedMatrix<ElemType>*> stripes;
                for (size_t w = 0; w < K; ++w)
                    stripes.push_back(&transport.ReceivedStripe(m_rank, w, i));
                Gpu(stripeQuantizer).StripeReduceAsync(stripes, m_rank, outStripeResidue, ownSlice, m_zeroThresholdFor1Bit);
            }
            else
            {
                // the aggregate lives in the own stripe of the input value (:347-353)
                Matrix<ElemType> aggGradStripe = call.inValues[i]->template GetWritableMatrix<ElemType>()->ColumnSlice(stripe.m_startCol, stripe.m_numCols);
                if (m_useQuantizationForSelfStripe)
                    stripeQuantizer.UnquantizeAsync(ownSlice, aggGradStripe, false); // (:410-416)
                for (size_t w = 0; w < K; ++w)
                {
                    if (w == m_rank)
                        continue;
                    QuantizedMatrix<ElemType>& received = const_cast<QuantizedMatrix<ElemType>&>(transport.ReceivedStripe(m_rank, w, i));
                    stripeQuantizer.UnquantizeAsync(received, aggGradStripe, true); // (:446-449)
                }
                stripeQuantizer.QuantizeAsync(aggGradStripe, inStripeResidue, ownSlice, outStripeResidue, m_zeroThresholdFor1Bit); // (:461-466)
            }
            if (!transport.StreamOrdered())
                fused ? Gpu(stripeQuantizer).WaitStripeReduceDone() : stripeQuantizer.WaitQuantizeAsyncDone(); // (:503)
            transport.PostAggregatedStripe(m_rank, i, st.quantizedGradients[i]->ColumnSlice(stripe.m_startCol, stripe.m_numCols));
        }
    }

    template <class ElemType>
    void FetchAndUnquantizeT(Call& call, StripeTransportT<ElemType>& transport, State<ElemType>& st)
    {
        const size_t K = NumWorkers();
        for (size_t i = 0; i < call.inValues.size(); ++i)
        {
            for (size_t j = 0; j < K; ++j)
            {
                if (j == m_rank)
                    continue;
                const auto stripe = AllReduceDistGradAggregator<ElemType>::GetStripeForNode(call.inValues[i]->GetNumCols(), j, K);
                if (stripe.m_numCols == 0)
                    continue;
                QuantizedMatrix<ElemType> dst = st.quantizedGradients[i]->ColumnSlice(stripe.m_startCol, stripe.m_numCols);
                transport.FetchAggregatedStripe(m_rank, j, i, dst, cntkq_stream(Gpu(*st.preAggregatedGradientQuantizers[i]).Handle()));
            }
            st.preAggregatedGradientQuantizers[i]->UnquantizeAsync(*st.quantizedGradients[i], *call.outputs[i]->template GetWritableMatrix<ElemType>(), false); // (:518)
        }
        for (size_t i = 0; i < call.inValues.size(); ++i)
            st.preAggregatedGradientQuantizers[i]->WaitUnquantizeAsyncDone(); // (:522-523)
    }

    StripeTransportT<float>& m_floatTransport;
    StripeTransportT<double>& m_doubleTransport;
    size_t m_rank;
    bool m_zeroThresholdFor1Bit;
    bool m_useQuantizationForSelfStripe;
    size_t m_numQuantizationBits;
    Options m_options;
    State<float> m_float;
    State<double> m_double;
};

// K communicators of one process on one GPU, driven in turn: worker r's argument lists are element r of every argument.
class InProcessCommunicators
{
public:
    InProcessCommunicators(size_t numWorkers, bool zeroThresholdFor1Bit, bool useQuantizationForSelfStripe, size_t numQuantizationBits,
                           QuantizedCommunicator::Options options = QuantizedCommunicator::Options())
        : m_floatTransport(numWorkers, true), m_doubleTransport(numWorkers, true)
    {
        for (size_t r = 0; r < numWorkers; ++r)
            m_workers.emplace_back(new QuantizedCommunicator(m_floatTransport, m_doubleTransport, r, zeroThresholdFor1Bit,
                                                             useQuantizationForSelfStripe, numQuantizationBits, options));
    }
    size_t NumWorkers() const { return m_workers.size(); }

    typedef std::vector<std::vector<NDArrayViewPtr>> PerWorker;

    // CNTK::QuantizedDistributedCommunicator::QuantizedAggregate, every worker's call at once (:64-96)
    void QuantizedAggregate(const PerWorker& inValues, PerWorker& valueQuantizationResidues, PerWorker& stripeQuantizationResidues,
                            PerWorker& aggregatedOutputs, PerWorker& newQuantizationResidues, PerWorker& newStripeQuantizationResidues)
    {
        const size_t K = m_workers.size();
        if (inValues.size() != K || valueQuantizationResidues.size() != K || stripeQuantizationResidues.size() != K ||
            aggregatedOutputs.size() != K || newQuantizationResidues.size() != K || newStripeQuantizationResidues.size() != K)
            throw std::invalid_argument("InProcessCommunicators: one argument list per worker");
        std::vector<QuantizedCommunicator::Call> calls;
        for (size_t r = 0; r < K; ++r)
            calls.push_back(m_workers[r]->Begin(inValues[r], valueQuantizationResidues[r], stripeQuantizationResidues[r], aggregatedOutputs[r],
                                                newQuantizationResidues[r], newStripeQuantizationResidues[r]));
        for (size_t r = 0; r < K; ++r)
            m_workers[r]->QuantizeAndPost(calls[r]);
        for (size_t r = 0; r < K; ++r)
            m_workers[r]->ReduceOwnStripes(calls[r]);
        for (size_t r = 0; r < K; ++r)
            m_workers[r]->FetchAndUnquantize(calls[r]);
    }

    // The plain sum of host values over the workers, each worker's buffer replaced by the sum
    // (MPICommunicatorImpl::AggregateInPlace, Source/CNTKv2LibraryDll/DistributedCommunicator.cpp:304-309, for CPU values;
    // the workers are added in ascending rank order).
    void AggregateInPlace(std::vector<std::vector<double>>& values)
    {
        if (values.size() != m_workers.size())
            throw std::invalid_argument("InProcessCommunicators: one argument list per worker");
        for (const auto& v : values)
            if (v.size() != values[0].size())
                throw std::logic_error("InProcessCommunicators: the workers' values differ in size");
        std::vector<double> sum = values[0];
        for (size_t r = 1; r < values.size(); ++r)
            for (size_t i = 0; i < sum.size(); ++i)
                sum[i] += values[r][i];
        for (auto& v : values)
            v = sum;
    }

    // (:51-62)
    void QuantizedAggregateInPlace(PerWorker& inValues, PerWorker& valueQuantizationResidues, PerWorker& stripeQuantizationResidues)
    {
        QuantizedAggregate(inValues, valueQuantizationResidues, stripeQuantizationResidues, inValues, valueQuantizationResidues,
                           stripeQuantizationResidues);
    }

private:
    InProcessTransportT<float> m_floatTransport;
    InProcessTransportT<double> m_doubleTransport;
    std::vector<std::unique_ptr<QuantizedCommunicator>> m_workers;
};

} // namespace cntk_amd
