// C++ test of the drop-in boundary through the host mirror classes, after the reference's own unit test
// (Tests/UnitTests/MathTests/MatrixQuantizerTests.cpp:239-472): for every bit width and, at 1 bit, both threshold
// modes, ten shapes x five iterations with the residual carried over and the output accumulated from the second
// iteration on. The checker is the CPU oracle (oracle/liboracle.so), fed the very inputs the device saw.
//
// Checks per iteration, as in the reference test:
//   * conservation:  in + prevResidual + prevOut == newResidual + newOut   within (hi - lo) * 1e-4       (:327-338)
//   * output and residual against the CPU checker within the same tolerance, with at most
//     max(1, 0.1 % of the elements) outliers ("may quantize to different integers")                     (:340-377)
// and, stricter than the reference: under the headers the device produced, codes and residual must equal the
// oracle's bit for bit, and unquantize must be bit-exact.
#include "../../cntk_amd/cpp/MatrixQuantizer.h"
#include "../../oracle/quantizer_oracle.h"

#include <cmath>
#include <cstdio>
#include <cstring>
#include <memory>
#include <random>
#include <string>
#include <vector>

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

// tolerances of the reference test (MatrixQuantizerTests.cpp:24-29)
static const float c_SinglePrecisionTolerance = 1e-4f;
static const double c_DoublePrecisionTolerance = 1e-8;
static const float c_SinglePrecisionGpuQuantizationTolerance = 1e-3f;
static const double c_DoublePrecisionGpuQuantizationTolerance = 1e-4;

// the CPU checker for either element type
template <class E> struct Oracle;
template <> struct Oracle<float>
{
    static int Quantize(const float* g, const float* r, size_t rows, size_t cols, void* q, size_t bits, float* rOut, int zt) { return oracle_quantize(g, r, rows, cols, q, bits, rOut, zt, 1); }
    static int Pack(const float* g, const float* r, size_t rows, size_t cols, void* q, size_t bits, float* rOut, int zt) { return oracle_pack_with_headers(g, r, rows, cols, q, bits, rOut, zt, 1); }
    static int Unquantize(const void* q, size_t rows, size_t cols, size_t bits, float* out, int add) { return oracle_unquantize(q, rows, cols, bits, out, add, 1); }
    static double Tolerance() { return c_SinglePrecisionTolerance; }
    static double OutlierShare() { return c_SinglePrecisionGpuQuantizationTolerance; }
};
template <> struct Oracle<double>
{
    static int Quantize(const double* g, const double* r, size_t rows, size_t cols, void* q, size_t bits, double* rOut, int zt) { return oracle_quantize_f64(g, r, rows, cols, q, bits, rOut, zt, 1); }
    static int Pack(const double* g, const double* r, size_t rows, size_t cols, void* q, size_t bits, double* rOut, int zt) { return oracle_pack_with_headers_f64(g, r, rows, cols, q, bits, rOut, zt, 1); }
    static int Unquantize(const void* q, size_t rows, size_t cols, size_t bits, double* out, int add) { return oracle_unquantize_f64(q, rows, cols, bits, out, add, 1); }
    static double Tolerance() { return c_DoublePrecisionTolerance; }
    static double OutlierShare() { return c_DoublePrecisionGpuQuantizationTolerance; }
};

template <class E>
static std::vector<E> RandomUniformT(size_t rows, size_t cols, E lo, E hi, unsigned long seed)
{
    std::mt19937_64 rng(seed);
    std::vector<E> a(rows * cols);
    for (auto& x : a)
        x = (E) (lo + (hi - lo) * ((rng() >> 11) * (1.0 / 9007199254740992.0)));
    return a;
}

static std::vector<float> RandomUniform(size_t rows, size_t cols, float lo, float hi, unsigned long seed)
{
    return RandomUniformT<float>(rows, cols, lo, hi, seed);
}

template <class E>
static void TestRunQuantization(size_t numBits, size_t numRows, size_t numCols, E rangeLow, E rangeHigh, int seed,
                                int numIterations, int deviceId, bool zeroThresholdFor1Bit, bool hostQuantizedMatrix)
{
    Matrix<E> inMatrix(numRows, numCols, deviceId);
    std::unique_ptr<MatrixQuantizerImpl<E>> quantizer(MatrixQuantizerImpl<E>::Create(deviceId, false /*useAsync*/));
    Matrix<E> residueMatrix(numRows, numCols, deviceId);
    Matrix<E> outMatrix(numRows, numCols, deviceId);
    const size_t numMatrixElems = inMatrix.GetNumElements();

    {
        // the initial residue and output are all zeros
        auto r = residueMatrix.CopyToArray(), o = outMatrix.CopyToArray();
        for (size_t i = 0; i < numMatrixElems; ++i)
            CHECK(r[i] == (E) 0 && o[i] == (E) 0, "fresh matrices must be zero");
    }

    for (int iterNum = 0; iterNum < numIterations; ++iterNum)
    {
        std::vector<E> in = RandomUniformT<E>(numRows, numCols, rangeLow, rangeHigh, (unsigned long) (seed + iterNum));
        inMatrix.SetValue(in.data());
        auto prevResidual = residueMatrix.CopyToArray();
        auto prevOut = outMatrix.CopyToArray();

        QuantizedMatrix<E> tempQuantizationBuffer(numRows, numCols, numBits, hostQuantizedMatrix ? CPUDEVICE : deviceId);
        quantizer->QuantizeAsync(inMatrix, residueMatrix, tempQuantizationBuffer, residueMatrix, zeroThresholdFor1Bit);
        quantizer->WaitQuantizeAsyncDone();
        quantizer->UnquantizeAsync(tempQuantizationBuffer, outMatrix, (iterNum > 0));
        quantizer->WaitUnquantizeAsyncDone();

        auto newResidual = residueMatrix.CopyToArray();
        auto newOut = outMatrix.CopyToArray();
        std::vector<char> packed = tempQuantizationBuffer.CopyToHost();

        double tolerance = 0.0;
        if (numBits != 8 * sizeof(E))
            tolerance = (double) (rangeHigh - rangeLow) * Oracle<E>::Tolerance();
        // a last-bit difference of the bounds moves a value by one code: 2^-32 of the range at 32 bits (double only)
        if (sizeof(E) == 8 && numBits == 32)
            tolerance = (double) (rangeHigh - rangeLow) * 1e-7;

        for (size_t i = 0; i < numMatrixElems; ++i)
            CHECK(std::fabs((double) (in[i] + prevResidual[i] + prevOut[i]) - (double) (newResidual[i] + newOut[i])) <=
                      tolerance + (sizeof(E) == 4 ? 1e-6 : 1e-14) * (double) (rangeHigh - rangeLow),
                  "conservation, element %zu", i);

        const size_t numIncorrectAllowed = std::max<size_t>(1, (size_t) (numMatrixElems * Oracle<E>::OutlierShare()));

        // the CPU checker on the same inputs
        std::vector<E> refResidual(numMatrixElems), refOut(prevOut.get(), prevOut.get() + numMatrixElems);
        std::vector<char> refPacked(packed.size());
        Oracle<E>::Quantize(in.data(), prevResidual.get(), numRows, numCols, refPacked.data(), numBits, refResidual.data(), zeroThresholdFor1Bit);
        Oracle<E>::Unquantize(refPacked.data(), numRows, numCols, numBits, refOut.data(), iterNum > 0);
        size_t numIncorrectOut = 0, numIncorrectResidual = 0;
        for (size_t i = 0; i < numMatrixElems; ++i)
        {
            if (std::fabs((double) newOut[i] - (double) refOut[i]) > tolerance && ++numIncorrectOut > numIncorrectAllowed)
                CHECK(false, "output differs from the CPU checker at %zu: %g vs %g", i, (double) newOut[i], (double) refOut[i]);
            if (std::fabs((double) newResidual[i] - (double) refResidual[i]) > tolerance && ++numIncorrectResidual > numIncorrectAllowed)
                CHECK(false, "residual differs from the CPU checker at %zu: %g vs %g", i, (double) newResidual[i], (double) refResidual[i]);
        }

        // stricter: bit-exact codes / residual under the device's own headers, bit-exact unquantize
        std::vector<char> exactPacked(packed);
        std::vector<E> exactResidual(numMatrixElems), exactOut(prevOut.get(), prevOut.get() + numMatrixElems);
        Oracle<E>::Pack(in.data(), prevResidual.get(), numRows, numCols, exactPacked.data(), numBits, exactResidual.data(), zeroThresholdFor1Bit);
        CHECK(std::memcmp(exactPacked.data(), packed.data(), packed.size()) == 0, "codes under the device's headers");
        CHECK(std::memcmp(exactResidual.data(), newResidual.get(), numMatrixElems * sizeof(E)) == 0, "residual under the device's headers");
        Oracle<E>::Unquantize(packed.data(), numRows, numCols, numBits, exactOut.data(), iterNum > 0);
        CHECK(std::memcmp(exactOut.data(), newOut.get(), numMatrixElems * sizeof(E)) == 0, "unquantize");
    }
}

template <class E>
static void TestQuantization(int deviceId, size_t numRows, size_t numCols, E rangeLow, E rangeHigh, int seed, int numIterations)
{
    // all power-of-two bit widths; 1 bit with and without zeroThresholdFor1Bit
    const size_t maxNumBits = 8 * sizeof(E);
    for (size_t numBits = 1; numBits <= maxNumBits; numBits *= 2)
        for (int i = 0; i < 2; ++i)
        {
            const bool zeroThresholdFor1Bit = (i == 1);
            if (numBits != 1 && zeroThresholdFor1Bit)
                continue;
            for (int host = 0; host < 2; ++host)
                TestRunQuantization<E>(numBits, numRows, numCols, rangeLow, rangeHigh, seed, numIterations, deviceId, zeroThresholdFor1Bit, host != 0);
        }
}

// the reference runs its ten cases for float and for double (MatrixQuantizerTests.cpp:406-431)
template <class E>
static void GPUMatrix1BitQuantize()
{
    const int dev = 0;
    TestQuantization<E>(dev, 25, 13, (E) -1.0, (E) +1.0, 2015, 5);
    TestQuantization<E>(dev, 25, 13, (E) -0.005, (E) +0.005, 2115, 5);
    TestQuantization<E>(dev, 13, 25, (E) -0.00001, (E) +0.00001, 2215, 5);
    TestQuantization<E>(dev, 13, 25, (E) -10.0, (E) +10.0, 2315, 5);
    TestQuantization<E>(dev, 25, 13, (E) -1.0, (E) +2.05, 2415, 5);
    TestQuantization<E>(dev, 489, 1, (E) -0.5, (E) +0.5, 2515, 5);
    TestQuantization<E>(dev, 1, 135, (E) -0.5, (E) +0.5, 2615, 5);
    TestQuantization<E>(dev, 89, 23, (E) -0.5, (E) +0.5, 2715, 5);
    TestQuantization<E>(dev, 15, 35, (E) -0.5, (E) +0.5, 2815, 5);
    TestQuantization<E>(dev, 100, 50, (E) -0.5, (E) +0.5, 2915, 5);
    // the sizes the reference test was first written with (:474-487)
    TestQuantization<E>(dev, 256, 135, (E) -1.0, (E) +2.05, 2415, 5);
    TestQuantization<E>(dev, 737, 373, (E) -0.5, (E) +0.5, 2915, 5);
    // the headline column height
    TestQuantization<E>(dev, 2048, 33, (E) -0.02, (E) +0.03, 3015, 3);
}

static void GPUMatrix1BitQuantizeFloat()
{
    GPUMatrix1BitQuantize<float>();
}

static void GPUMatrix1BitQuantizeDouble()
{
    GPUMatrix1BitQuantize<double>();
}

// A gradient set through the batched calls gives the bytes of the per-matrix calls.
static void BatchEqualsPerMatrix()
{
    const size_t shapes[][2] = {{147, 64}, {64, 64}, {576, 64}, {1, 5}, {429, 37}, {2048, 33}, {2304, 5}, {9304, 1}, {1000, 1}, {512, 100}};
    const size_t numBits[] = {1, 4};
    for (size_t nb : numBits)
    {
        auto* gpu = new MatrixQuantizerGPU<float>(0, true);
        std::unique_ptr<MatrixQuantizerImpl<float>> owner(gpu);
        std::vector<std::unique_ptr<Matrix<float>>> in, res1, res2, out1, out2;
        std::vector<std::unique_ptr<QuantizedMatrix<float>>> q1, q2;
        for (const auto& s : shapes)
        {
            in.emplace_back(new Matrix<float>(s[0], s[1], 0));
            std::vector<float> host = RandomUniform(s[0], s[1], -0.01f, 0.02f, 77 + s[0]);
            in.back()->SetValue(host.data());
            res1.emplace_back(new Matrix<float>(s[0], s[1], 0));
            res2.emplace_back(new Matrix<float>(s[0], s[1], 0));
            out1.emplace_back(new Matrix<float>(s[0], s[1], 0));
            out2.emplace_back(new Matrix<float>(s[0], s[1], 0));
            q1.emplace_back(new QuantizedMatrix<float>(s[0], s[1], nb, 0));
            q2.emplace_back(new QuantizedMatrix<float>(s[0], s[1], nb, 0));
        }
        std::vector<MatrixQuantizerGPU<float>::QuantizeItem> qi;
        std::vector<MatrixQuantizerGPU<float>::UnquantizeItem> ui;
        for (size_t i = 0; i < in.size(); ++i)
        {
            gpu->QuantizeAsync(*in[i], *res1[i], *q1[i], *res1[i], nb == 1);
            qi.push_back({in[i].get(), res2[i].get(), q2[i].get(), res2[i].get()});
            ui.push_back({q2[i].get(), out2[i].get()});
        }
        gpu->QuantizeBatchAsync(qi, nb == 1);
        gpu->WaitQuantizeAsyncDone();
        for (size_t i = 0; i < in.size(); ++i)
            gpu->UnquantizeAsync(*q1[i], *out1[i]);
        gpu->UnquantizeBatchAsync(ui);
        gpu->WaitUnquantizeAsyncDone();
        for (size_t i = 0; i < in.size(); ++i)
        {
            const size_t n = in[i]->GetNumElements();
            CHECK(q1[i]->CopyToHost() == q2[i]->CopyToHost(), "batched codes, matrix %zu", i);
            CHECK(std::memcmp(res1[i]->CopyToArray().get(), res2[i]->CopyToArray().get(), n * sizeof(float)) == 0, "batched residual, matrix %zu", i);
            CHECK(std::memcmp(out1[i]->CopyToArray().get(), out2[i]->CopyToArray().get(), n * sizeof(float)) == 0, "batched output, matrix %zu", i);
        }
    }
}

static void ErrorBehaviour()
{
    bool threw = false;
    try { QuantizedMatrix<float> q(8, 8, 3, 0); } catch (const std::logic_error&) { threw = true; }
    CHECK(threw, "nbits = 3 must be a logic error");
    threw = false;
    try { std::unique_ptr<MatrixQuantizerImpl<float>> q(MatrixQuantizerImpl<float>::Create(CPUDEVICE, false)); } catch (const std::runtime_error&) { threw = true; }
    CHECK(threw, "no CPU quantizer");
    std::unique_ptr<MatrixQuantizerImpl<float>> q(MatrixQuantizerImpl<float>::Create(0, true));
    Matrix<float> a(8, 4, 0), b(8, 5, 0);
    QuantizedMatrix<float> qa(8, 4, 1, 0);
    threw = false;
    try { q->QuantizeAsync(a, b, qa, a, false); } catch (const std::invalid_argument&) { threw = true; }
    CHECK(threw, "dimension mismatch");
    threw = false;
    try { q->UnquantizeAsync(qa, b); } catch (const std::invalid_argument&) { threw = true; }
    CHECK(threw, "dimension mismatch on unquantize");
    CHECK(q->GetDeviceId() == 0, "device id");
    // residual-owning wrapper: ResetResidue really clears
    MatrixQuantizer<float> mq(64, 8, 0, true);
    Matrix<float> g(64, 8, 0);
    g.SetValue(0.25f);
    QuantizedMatrix<float> qm(64, 8, 1, 0);
    mq.QuantizeAsync(g, qm, true);
    mq.WaitQuantizeAsyncDone();
    mq.ResetResidue();
    auto r = mq.GetResidualMatrix().CopyToArray();
    for (size_t i = 0; i < 64 * 8; ++i)
        CHECK(r[i] == 0.0f, "ResetResidue");
}

// QuantizedMatrix::Print on the hand example {0.1, -0.2, 0.3, -0.4, 0.05} (1 bit, mean threshold): bounds -0.462 / 0.402,
// codes 1 0 1 0 1, reconstructed values lower + (code + 0.5) * (upper - lower) / 2 ... written to a temporary file.
template <class E>
static void PrintOne()
{
    const E host[5] = {(E) 0.1, (E) -0.2, (E) 0.3, (E) -0.4, (E) 0.05};
    Matrix<E> g(5, 1, 0);
    g.SetValue(host);
    MatrixQuantizer<E> mq(5, 1, 0, false);
    QuantizedMatrix<E> q(5, 1, 1, 0);
    mq.QuantizeAsync(g, q, false);
    mq.WaitQuantizeAsyncDone();
    FILE* f = std::tmpfile();
    CHECK(f != nullptr, "tmpfile");
    if (f == nullptr)
        return;
    q.Print("grad", 0, 4, 0, 0, f);
    std::rewind(f);
    std::string text;
    char buf[256];
    while (std::fgets(buf, sizeof buf, f) != nullptr)
        text += buf;
    std::fclose(f);
    CHECK(text.find("###### grad (5, 1) ######") != std::string::npos, "title: %s", text.c_str());
    CHECK(text.find("Print Range (0:4, 0:0)") != std::string::npos, "range");
    CHECK(text.find("Lower=-0.462") != std::string::npos && text.find("Upper=0.402") != std::string::npos, "bounds: %s", text.c_str());
    // five element lines: code then value in parentheses; low level -0.246, high level 0.186
    const char* expect[5] = {"1 (0.18", "0 (-0.24", "1 (0.18", "0 (-0.24", "1 (0.18"};
    size_t pos = text.find("Upper=");
    for (int i = 0; i < 5; ++i)
    {
        const size_t at = text.find(expect[i], pos);
        CHECK(at != std::string::npos, "element %d: %s", i, text.c_str());
        if (at == std::string::npos)
            break;
        pos = at + 1;
    }
    bool threw = false;
    try { q.Print(nullptr, 0, 5, 0, 0, stderr); } catch (const std::invalid_argument&) { threw = true; }
    CHECK(threw, "Print: index out of range");
}

static void PrintPackedMatrix()
{
    PrintOne<float>();
    PrintOne<double>();
}

int main()
{
    try
    {
        GPUMatrix1BitQuantizeFloat();
        std::printf("Test case GPUMatrixSuite/GPUMatrix1BitQuantizeFloat %s\n", g_failures ? "has FAILED" : "has passed");
        int before = g_failures;
        GPUMatrix1BitQuantizeDouble();
        std::printf("Test case GPUMatrixSuite/GPUMatrix1BitQuantizeDouble %s\n", g_failures != before ? "has FAILED" : "has passed");
        before = g_failures;
        BatchEqualsPerMatrix();
        std::printf("Test case GPUMatrixSuite/QuantizerBatchEqualsPerMatrix %s\n", g_failures != before ? "has FAILED" : "has passed");
        before = g_failures;
        ErrorBehaviour();
        std::printf("Test case GPUMatrixSuite/QuantizerErrorBehaviour %s\n", g_failures != before ? "has FAILED" : "has passed");
        before = g_failures;
        PrintPackedMatrix();
        std::printf("Test case GPUMatrixSuite/QuantizedMatrixPrint %s\n", g_failures != before ? "has FAILED" : "has passed");
    }
    catch (const std::exception& e)
    {
        std::fprintf(stderr, "unexpected exception: %s\n", e.what());
        return 2;
    }
    std::fflush(stdout);
    return g_failures ? 1 : 0;
}
