// Tests of the C++ host layer, written after the reference's own suites
// (ILGPU.Algorithms.Tests: RadixSortExtensionTests.tt, ScanExtensionTests.tt,
// ReductionExtensionTests.tt, HistogramTests.tt, TempViewManagerTests.cs):
// same sequences, sizes, call pattern (create once, invoke with a stream,
// synchronise, verify) and expectations computed on the host.
//
//   host_api_tests            all tests (needs a GPU)
//   host_api_tests --host     only the tests that touch no device
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "../../ilgpu_amd/host/ilgpu_hip_algorithms.hpp"

using namespace ilgpu;
using namespace ilgpu::Algorithms;
namespace RSO = ilgpu::RadixSortOperations;
namespace SRO = ilgpu::ScanReduceOperations;

static int g_failed = 0, g_run = 0;
#define CHECK(cond)                                                            \
  do {                                                                         \
    if (!(cond)) {                                                             \
      std::printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);          \
      ++g_failed;                                                              \
    }                                                                          \
  } while (0)
#define EXPECT_THROW(stmt, Ex)                                                 \
  do {                                                                         \
    bool caught = false;                                                       \
    try { stmt; } catch (const Ex&) { caught = true; } catch (...) {}          \
    if (!caught) {                                                             \
      std::printf("  FAILED %s:%d: expected %s\n", __FILE__, __LINE__, #Ex);   \
      ++g_failed;                                                              \
    }                                                                          \
  } while (0)
#define RUN(fn)                                                                \
  do {                                                                         \
    std::printf("[ RUN  ] %s\n", #fn);                                         \
    std::fflush(stdout);                                                       \
    ++g_run;                                                                   \
    fn;                                                                        \
  } while (0)

// ArraySizes (Generic/ConfigurationBase.tt:80)
static const int kArraySizes[] = {1, 31, 33, 127, 1027};

// ITestSequencer (Generic/AlgorithmsTestData.tt:74-96)
template <typename T> std::vector<T> ComputeSequence(T start, T step, int length) {
  std::vector<T> s((size_t)length);
  s[0] = start;
  for (int i = 1; i < length; ++i) s[i] = (T)(s[i - 1] + step);
  return s;
}
template <typename T> std::vector<T> ComputeInvertedSequence(T start, T step, int length) {
  std::vector<T> s((size_t)length);
  s[length - 1] = start;
  for (int i = length - 2; i >= 0; --i) s[i] = (T)(s[i + 1] + step);
  return s;
}
template <typename T> bool Verify(const std::vector<T>& got, const std::vector<T>& expected) {
  return got.size() >= expected.size() &&
         std::memcmp(got.data(), expected.data(), expected.size() * sizeof(T)) == 0;
}

// ---- RadixSortExtensionTests -------------------------------------------------
template <typename T, typename TAsc, typename TDesc> void RadixTests(Accelerator& accl) {
  for (int length : kArraySizes) {
    auto stream = accl.CreateStream();
    const auto seq = ComputeSequence<T>(0, 1, length);
    const auto inv = ComputeInvertedSequence<T>(0, 1, length);
    const Index1D tempSize = ComputeRadixSortTempStorageSize<T, TAsc>(accl, length);
    auto tmp = accl.Allocate1D<int32_t>(tempSize);
    {  // RadixWorstCaseAscending (:144-187)
      auto input = accl.Allocate1D<T>(length);
      input->CopyFromCPU(*stream, inv);
      auto radixSort = CreateRadixSort<T, Stride1D::Dense, TAsc>(accl);
      radixSort(*stream, input->View(), tmp->View());
      stream->Synchronize();
      CHECK(Verify(input->GetAsArray1D(), seq));
    }
    {  // RadixBestCaseAscending (:189-230)
      auto input = accl.Allocate1D<T>(length);
      input->CopyFromCPU(*stream, seq);
      CreateRadixSort<T, Stride1D::Dense, TAsc>(accl)(*stream, input->View(), tmp->View());
      stream->Synchronize();
      CHECK(Verify(input->GetAsArray1D(), seq));
    }
    {  // RadixWorstCaseDescending
      auto input = accl.Allocate1D<T>(length);
      input->CopyFromCPU(*stream, seq);
      CreateRadixSort<T, Stride1D::Dense, TDesc>(accl)(*stream, input->View(), tmp->View());
      stream->Synchronize();
      CHECK(Verify(input->GetAsArray1D(), inv));
    }
    {  // RadixProviderWorstCaseAscending (:232-317)
      auto input = accl.Allocate1D<T>(length);
      input->CopyFromCPU(*stream, inv);
      auto provider = CreateRadixSortProvider<T, TAsc>(accl, length);
      auto sortUsingProvider = provider->template CreateRadixSort<T, Stride1D::Dense, TAsc>();
      sortUsingProvider(*stream, input->View());
      stream->Synchronize();
      CHECK(Verify(input->GetAsArray1D(), seq));
    }
    {  // RadixSortPairsAscending (:319-365): values == keys
      auto keys = accl.Allocate1D<T>(length);
      auto values = accl.Allocate1D<T>(length);
      keys->CopyFromCPU(*stream, inv);
      values->CopyFromCPU(*stream, inv);
      auto sortPairs = CreateRadixSortPairs<T, Stride1D::Dense, T, Stride1D::Dense, TAsc>(accl);
      auto tmpPairs = accl.Allocate1D<int32_t>(
          ComputeRadixSortPairsTempStorageSize<T, T, TAsc>(accl, length));
      sortPairs(*stream, keys->View(), values->View(), tmpPairs->View());
      stream->Synchronize();
      CHECK(Verify(keys->GetAsArray1D(), seq));
      CHECK(Verify(values->GetAsArray1D(), seq));
    }
    // RadixConstCase (:370-432): start in {0, 1, -1}, step 0
    for (int start : {0, 1, -1}) {
      if (std::is_unsigned<T>::value && start < 0) continue;
      const auto constant = ComputeSequence<T>((T)start, 0, length);
      auto input = accl.Allocate1D<T>(length);
      input->CopyFromCPU(*stream, constant);
      CreateRadixSort<T, Stride1D::Dense, TAsc>(accl)(*stream, input->View(), tmp->View());
      stream->Synchronize();
      CHECK(Verify(input->GetAsArray1D(), constant));
    }
  }
}

static void RadixSortSequencerPairs(Accelerator& accl) {
  // CreateRadixSortPairs with an index sequencer (RadixSortExtensions.cs:1017-1074)
  const int n = 5003;
  std::vector<uint32_t> keys((size_t)n);
  for (int i = 0; i < n; ++i) keys[i] = (uint32_t)((i * 2654435761u) >> 24);  // many ties
  std::vector<int32_t> order((size_t)n);
  for (int i = 0; i < n; ++i) order[i] = i;
  std::stable_sort(order.begin(), order.end(),
                   [&](int a, int b) { return keys[a] < keys[b]; });
  auto dKeys = accl.Allocate1D<uint32_t>(keys);
  auto dValues = accl.Allocate1D<int32_t>(n);
  auto tmp = accl.Allocate1D<int32_t>(
      ComputeRadixSortPairsTempStorageSize<uint32_t, int32_t, RSO::AscendingUInt32>(accl, n));
  auto sort = CreateRadixSortPairsWithSequencer<uint32_t, Stride1D::Dense, int32_t,
                                                Stride1D::Dense, Sequencers::Int32Sequencer,
                                                RSO::AscendingUInt32>(accl);
  sort(accl.DefaultStream(), dKeys->View(), dValues->View(), Sequencers::Int32Sequencer(),
       tmp->View());
  accl.Synchronize();
  CHECK(Verify(dValues->GetAsArray1D(), order));
}

// A strided key view (Stride1D.General{3}): sorted in place, gaps untouched; the
// temp comes from the sizing overload that takes the stride.
static void RadixSortStrided(Accelerator& accl) {
  const int n = 1027, stride = 3;
  std::vector<uint32_t> host((n - 1) * stride + 1, 0xABABABABu);
  std::vector<uint32_t> keys(n);
  for (int i = 0; i < n; ++i) keys[i] = host[(size_t)i * stride] = (uint32_t)((i * 2654435761u) >> 7);
  auto buf = accl.Allocate1D<uint32_t>((int64_t)host.size());
  buf->CopyFromCPU(host);
  ArrayView1D<uint32_t, Stride1D::General> view(buf->View(), n, Stride1D::General{stride});
  auto sort = CreateRadixSort<uint32_t, Stride1D::General, RSO::AscendingUInt32>(accl);
  auto dense_tmp = accl.Allocate1D<int32_t>(
      (int64_t)ComputeRadixSortTempStorageSize<uint32_t, RSO::AscendingUInt32>(accl, n));
  EXPECT_THROW(sort(accl.DefaultStream(), view, dense_tmp->View()), ArgumentOutOfRangeException);
  auto tmp = accl.Allocate1D<int32_t>(
      (int64_t)ComputeRadixSortTempStorageSize<uint32_t, RSO::AscendingUInt32>(accl, n, stride));
  sort(accl.DefaultStream(), view, tmp->View());
  accl.Synchronize();
  auto got = buf->GetAsArray1D();
  std::sort(keys.begin(), keys.end());
  bool ok = true;
  for (size_t i = 0; i < got.size(); ++i)
    ok = ok && got[i] == (i % stride == 0 ? keys[i / stride] : 0xABABABABu);
  CHECK(ok);
}

static void RadixSortErrors(Accelerator& accl) {
  auto sort = CreateRadixSort<int32_t, Stride1D::Dense, RSO::AscendingInt32>(accl);
  auto data = accl.Allocate1D<int32_t>(64);
  auto tmp = accl.Allocate1D<int32_t>(
      ComputeRadixSortTempStorageSize<int32_t, RSO::AscendingInt32>(accl, 64));
  auto& s = accl.DefaultStream();
  EXPECT_THROW(sort(s, ArrayView<int32_t>(), tmp->View()), ArgumentNullException);
  EXPECT_THROW(sort(s, data->View(), ArrayView<int32_t>()), ArgumentNullException);
  EXPECT_THROW(sort(s, data->View(), tmp->View().SubView(0, 4)), ArgumentOutOfRangeException);
  auto pairs = CreateRadixSortPairs<int32_t, Stride1D::Dense, int32_t, Stride1D::Dense,
                                    RSO::AscendingInt32>(accl);
  auto vals = accl.Allocate1D<int32_t>(32);
  EXPECT_THROW(pairs(s, data->View(), vals->View(), tmp->View()), ArgumentOutOfRangeException);
  EXPECT_THROW(RadixSortProvider(accl, 0), ArgumentOutOfRangeException);
}

// ---- ScanExtensionTests -------------------------------------------------------
template <typename T, typename TOp>
std::vector<T> CalcValues(const std::vector<T>& seq, ScanKind kind) {
  // ScanExtensionTests.tt:286-305
  std::vector<T> out(seq.size());
  T acc = TOp::Identity();
  for (size_t i = 0; i < seq.size(); ++i) {
    T next;
    if (TOp::Op == ILGPU_HIP_OP_ADD) next = (T)(acc + seq[i]);
    else if (TOp::Op == ILGPU_HIP_OP_MAX) next = std::max(acc, seq[i]);
    else next = std::min(acc, seq[i]);
    out[i] = kind == ScanKind::Inclusive ? next : acc;
    acc = next;
  }
  return out;
}

template <typename T, typename TOp> void ScanTests(Accelerator& accl, int maxLength) {
  for (int length : kArraySizes) {
    if (length > maxLength) continue;  // floats: :52
    for (int variant = 0; variant < 3; ++variant) {
      // ascending (0,1), constant (1,0), descending (length,-1) as inverted ascending
      std::vector<T> seq = variant == 0   ? ComputeSequence<T>(0, 1, length)
                           : variant == 1 ? ComputeSequence<T>(1, 0, length)
                                          : ComputeInvertedSequence<T>(1, 1, length);
      for (ScanKind kind : {ScanKind::Inclusive, ScanKind::Exclusive}) {
        auto input = accl.Allocate1D<T>(seq);
        auto output = accl.Allocate1D<T>(length);
        auto scan = CreateScan<T, Stride1D::General, Stride1D::General, TOp>(accl, kind);
        auto tmp = accl.Allocate1D<int32_t>((int64_t)ComputeScanTempStorageSize<T>(accl, length));
        // the reference always goes through AsGeneral() views (:148-154)
        ArrayView1D<T> in(input->View()), out(output->View());
        scan(accl.DefaultStream(), in.AsGeneral(), out.AsGeneral(), tmp->View());
        accl.Synchronize();
        CHECK(Verify(output->GetAsArray1D(), CalcValues<T, TOp>(seq, kind)));
      }
    }
  }
}

static void ScanErrors(Accelerator& accl) {
  auto scan = CreateScan<int32_t, Stride1D::Dense, Stride1D::Dense, SRO::AddInt32>(
      accl, ScanKind::Inclusive);
  auto in = accl.Allocate1D<int32_t>(100);
  auto out = accl.Allocate1D<int32_t>(100);
  auto tmp = accl.Allocate1D<int32_t>((int64_t)ComputeScanTempStorageSize<int32_t>(accl, 100));
  auto& s = accl.DefaultStream();
  EXPECT_THROW(scan(s, ArrayView<int32_t>(), out->View(), tmp->View()), ArgumentNullException);
  EXPECT_THROW(scan(s, in->View(), ArrayView<int32_t>(), tmp->View()), ArgumentNullException);
  EXPECT_THROW(scan(s, in->View(), out->View().SubView(0, 50), tmp->View()),
               ArgumentOutOfRangeException);
  EXPECT_THROW(scan(s, in->View(), out->View(), ArrayView<int32_t>()), ArgumentNullException);
  // Stride1D.General with an element stride of 2: every other element.
  {
    std::vector<int32_t> host(100);
    for (int i = 0; i < 100; ++i) host[i] = i % 2 == 0 ? i / 2 + 1 : -1000;
    in->CopyFromCPU(host);
    out->CopyFromCPU(std::vector<int32_t>(100, 7));
    ArrayView1D<int32_t, Stride1D::General> strided(in->View(), 50, Stride1D::General{2});
    auto gscan = CreateScan<int32_t, Stride1D::General, Stride1D::Dense, SRO::AddInt32>(
        accl, ScanKind::Inclusive);
    gscan(s, strided, out->View(), tmp->View());
    accl.Synchronize();
    auto got = out->GetAsArray1D();
    bool ok = true;
    for (int i = 0; i < 50; ++i) ok = ok && got[i] == (i + 1) * (i + 2) / 2;
    for (int i = 50; i < 100; ++i) ok = ok && got[i] == 7;  // beyond the 50 results
    CHECK(ok);
  }
  // provider variant
  auto provider = CreateScanProvider<int32_t>(accl, 100);
  auto buffered = provider->CreateScan<int32_t, Stride1D::Dense, Stride1D::Dense, SRO::AddInt32>(
      ScanKind::Exclusive);
  in->CopyFromCPU(std::vector<int32_t>(100, 2));
  buffered(s, in->View(), out->View());
  accl.Synchronize();
  auto got = out->GetAsArray1D();
  CHECK(got[0] == 0 && got[99] == 198);
}

// ---- UniqueExtensionTests (UniqueExtensionTests.tt:36-90) -----------------------
template <typename T> void UniqueTests(Accelerator& accl) {
  namespace CO = ilgpu::ComparisonOperations;
  for (int repeat : {1, 317, 1025}) {
    for (int length : {1025, 70000}) {
      std::vector<T> input((size_t)length), expected;
      for (int i = 0; i < length; ++i) input[i] = (T)(i / repeat + 1);
      for (const T& e : input)
        if (expected.empty() || expected.back() != e) expected.push_back(e);
      auto buf = accl.Allocate1D<T>(length);
      buf->CopyFromCPU(input);
      const int64_t result =
          Unique<T, CO::Comparison<T>>(accl, accl.DefaultStream(), buf->View());
      CHECK(result == (int64_t)expected.size());
      CHECK(Verify(buf->GetAsArray1D(), expected));
    }
  }
}
static void UniqueErrors(Accelerator& accl) {
  namespace CO = ilgpu::ComparisonOperations;
  auto unique = CreateUnique<int32_t, CO::ComparisonInt32>(accl);
  auto in = accl.Allocate1D<int32_t>(100);
  auto out = accl.Allocate1D<int64_t>(1);
  auto tmp = accl.Allocate1D<int32_t>(ComputeUniqueTempStorageSize<int32_t>(accl, 100));
  auto& s = accl.DefaultStream();
  EXPECT_THROW(unique(s, ArrayView<int32_t>(), out->View(), tmp->View()), ArgumentNullException);
  EXPECT_THROW(unique(s, in->View(), ArrayView<int64_t>(), tmp->View()), ArgumentNullException);
  EXPECT_THROW(unique(s, in->View(), out->View(), ArrayView<int32_t>()), ArgumentNullException);
  EXPECT_THROW(unique(s, in->View(), out->View(), tmp->View().SubView(0, 1)),
               ArgumentOutOfRangeException);
}

// ---- SequencerTests (SequencerTests.tt:56-200), InitializeTests, ReorderExtensionTests ----
template <typename T, typename TSequencer> void SequencerTests(Accelerator& accl) {
  for (int length : kArraySizes) {
    auto buf = accl.Allocate1D<T>(length);
    auto stream = accl.CreateStream();
    ArrayView1D<T, Stride1D::Dense> view(buf->View());
    Sequence(accl, *stream, view, TSequencer());
    stream->Synchronize();
    std::vector<T> expected((size_t)length);
    for (int i = 0; i < length; ++i) expected[i] = (T)i;
    CHECK(Verify(buf->GetAsArray1D(), expected));
    RepeatedSequence(accl, *stream, view, 2, TSequencer());
    stream->Synchronize();
    for (int i = 0; i < length; ++i) expected[i] = (T)(i % 2);
    CHECK(Verify(buf->GetAsArray1D(), expected));
    BatchedSequence(accl, *stream, view, 2, TSequencer());
    stream->Synchronize();
    for (int i = 0; i < length; ++i) expected[i] = (T)(i / 2);
    CHECK(Verify(buf->GetAsArray1D(), expected));
    RepeatedBatchedSequence(accl, *stream, view, 2, 2, TSequencer());
    stream->Synchronize();
    for (int i = 0; i < length; ++i) expected[i] = (T)((i / 2) % 2);
    CHECK(Verify(buf->GetAsArray1D(), expected));
    EXPECT_THROW(RepeatedSequence(accl, *stream, view, 0, TSequencer()),
                 ArgumentOutOfRangeException);
    EXPECT_THROW(BatchedSequence(accl, *stream, view, 0, TSequencer()),
                 ArgumentOutOfRangeException);
  }
}
template <typename T> void InitializeAndReorderTests(Accelerator& accl) {
  for (int length : kArraySizes) {
    auto buf = accl.Allocate1D<T>(length);
    auto target = accl.Allocate1D<T>(length);
    auto order = accl.Allocate1D<Index1D>(length);
    auto& s = accl.DefaultStream();
    Initialize(accl, s, buf->View(), (T)42);
    accl.Synchronize();
    CHECK(Verify(buf->GetAsArray1D(), std::vector<T>((size_t)length, (T)42)));
    // reverse through Reorder
    const auto seq = ComputeSequence<T>(0, 1, length);
    std::vector<Index1D> rev((size_t)length);
    for (int i = 0; i < length; ++i) rev[i] = length - 1 - i;
    buf->CopyFromCPU(seq);
    order->CopyFromCPU(rev);
    Reorder(accl, s, buf->View(), target->View(), order->View());
    accl.Synchronize();
    CHECK(Verify(target->GetAsArray1D(), ComputeInvertedSequence<T>(0, 1, length)));
    if (length > 1) {
      EXPECT_THROW(Reorder(accl, s, buf->View(), target->View(), order->View().SubView(0, length - 1)),
                   ArgumentOutOfRangeException);
      EXPECT_THROW(Reorder(accl, s, buf->View(), target->View().SubView(0, length - 1), order->View()),
                   ArgumentOutOfRangeException);
    }
    EXPECT_THROW(Initialize(accl, s, ArrayView<T>(), (T)1), ArgumentNullException);
  }
}

// ---- TransformerExtensionTests, ReorderExtensionTests (transformers) ---------------
// TransformerExtensionTests.tt:66-134 with the closed-set stand-ins for
// IntToNegIntTransformer, IntToLongTransformer and UInt32ToBitCompInt32Transformer.
void TransformTests(Accelerator& accl) {
  auto& s = accl.DefaultStream();
  for (int length : kArraySizes) {
    const auto seq = ComputeSequence<int32_t>(42, 0, length);
    auto input = accl.Allocate1D<int32_t>(seq);
    auto output = accl.Allocate1D<int32_t>(length);
    Transform<int32_t, int32_t>(accl, s, input->View(), output->View(),
                                NegateTransformer<int32_t>());
    accl.Synchronize();
    CHECK(Verify(output->GetAsArray1D(), std::vector<int32_t>((size_t)length, -42)));

    auto wide = accl.Allocate1D<int64_t>(length);
    auto transformer = CreateTransformer<int32_t, int64_t, ConvertTransformer<int32_t, int64_t>>(accl);
    transformer(s, input->View(), wide->View(), ConvertTransformer<int32_t, int64_t>());
    accl.Synchronize();
    CHECK(Verify(wide->GetAsArray1D(), std::vector<int64_t>((size_t)length, 42)));

    const auto useq = ComputeSequence<uint32_t>(0, 1, length);
    auto uinput = accl.Allocate1D<uint32_t>(useq);
    Transform<uint32_t, int32_t>(accl, s, uinput->View(), output->View(),
                                 BitComplementTransformer<uint32_t, int32_t>());
    accl.Synchronize();
    std::vector<int32_t> comp((size_t)length);
    for (int i = 0; i < length; ++i) comp[i] = (int32_t)~useq[i];
    CHECK(Verify(output->GetAsArray1D(), comp));

    // in place (TransformExtensions.cs:377-393)
    Transform<int32_t>(accl, s, input->View(), MultiplyTransformer<int32_t>{3});
    accl.Synchronize();
    CHECK(Verify(input->GetAsArray1D(), std::vector<int32_t>((size_t)length, 126)));

    if (length > 1) {
      EXPECT_THROW((Transform<int32_t, int32_t>(accl, s, input->View(),
                                                 output->View().SubView(0, length - 1),
                                                 NegateTransformer<int32_t>())),
                   ArgumentOutOfRangeException);
    }
    EXPECT_THROW((Transform<int32_t, int32_t>(accl, s, ArrayView<int32_t>(), output->View(),
                                               NegateTransformer<int32_t>())),
                 ArgumentNullException);
  }
}

// TransformerExtensionTests.tt:136-162: Index1D -> T.
template <typename T> void CastFromIndexTests(Accelerator& accl) {
  for (int length : kArraySizes) {
    const auto seq = ComputeSequence<Index1D>(0, 1, length);
    auto input = accl.Allocate1D<Index1D>(seq);
    auto output = accl.Allocate1D<T>(length);
    Transform<Index1D, T>(accl, accl.DefaultStream(), input->View(), output->View(),
                          ConvertTransformer<Index1D, T>());
    accl.Synchronize();
    std::vector<T> expected((size_t)length);
    for (int i = 0; i < length; ++i) expected[i] = (T)seq[i];
    CHECK(Verify(output->GetAsArray1D(), expected));
  }
}

// ReorderExtensionTests.tt:160-200 (<T>Mul2, reversed order) and :240-290 (widening).
template <typename T> void ReorderTransformTests(Accelerator& accl) {
  auto& s = accl.DefaultStream();
  for (int length : kArraySizes) {
    for (int variant = 0; variant < 3; ++variant) {
      const auto seq = variant == 0 ? ComputeSequence<T>(0, 0, length)
                     : variant == 1 ? ComputeSequence<T>(1, 0, length)
                                    : ComputeSequence<T>(0, 1, length);
      std::vector<Index1D> rev((size_t)length);
      for (int i = 0; i < length; ++i) rev[i] = length - 1 - i;
      auto input = accl.Allocate1D<T>(seq);
      auto order = accl.Allocate1D<Index1D>(rev);
      auto output = accl.Allocate1D<T>(length);
      ReorderTransform<T>(accl, s, input->View(), output->View(), order->View(),
                          MultiplyTransformer<T>{2});
      accl.Synchronize();
      std::vector<T> expected((size_t)length);   // CalcValues: result[order[i]] = f(input[i])
      for (int i = 0; i < length; ++i) expected[rev[i]] = (T)(seq[i] * 2);
      CHECK(Verify(output->GetAsArray1D(), expected));
    }
  }
}

// ---- ReductionExtensionTests ----------------------------------------------------
template <typename T, typename TOp> void ReduceTests(Accelerator& accl, int maxLength) {
  for (int length : kArraySizes) {
    if (length > maxLength) continue;
    for (int variant = 0; variant < 2; ++variant) {
      const auto seq = variant == 0 ? ComputeSequence<T>(0, 1, length)
                                    : ComputeSequence<T>(1, 0, length);
      const T expected = CalcValues<T, TOp>(seq, ScanKind::Inclusive).back();  // left fold (:205-212)
      auto input = accl.Allocate1D<T>(seq);
      // value-returning overload with its cached output (:119-150)
      const T got = Reduce<T, TOp>(accl, accl.DefaultStream(), input->View());
      CHECK(got == expected);
      // explicit output view (:152-196); output[0] is overwritten
      auto output = accl.Allocate1D<T>(std::vector<T>{(T)77, (T)78});
      Reduce<T, TOp>(accl, accl.DefaultStream(), input->View(), output->View());
      accl.Synchronize();
      auto o = output->GetAsArray1D();
      CHECK(o[0] == expected && o[1] == (T)78);
    }
  }
}

static void ReduceErrors(Accelerator& accl) {
  auto reduce = CreateReduction<float, Stride1D::Dense, SRO::AddFloat>(accl);
  auto in = accl.Allocate1D<float>(10);
  auto out = accl.Allocate1D<float>(1);
  auto& s = accl.DefaultStream();
  EXPECT_THROW(reduce(s, ArrayView<float>(), out->View()), ArgumentNullException);
  EXPECT_THROW(reduce(s, in->View(), ArrayView<float>()), ArgumentNullException);
}

// One delegate invoked on two streams at once: the reference's delegate has no
// hidden state (ReductionExtensions.cs:135-167), so neither may ours.  Large
// inputs keep both reductions in flight together; every invocation must give
// its own input's sum.
static void ReduceOnTwoStreams(Accelerator& accl) {
  auto reduce = CreateReduction<int64_t, Stride1D::Dense, SRO::AddInt64>(accl);
  const int length = 1 << 22;
  std::vector<int64_t> a((size_t)length), b((size_t)length);
  int64_t sumA = 0, sumB = 0;
  for (int i = 0; i < length; ++i) {
    a[i] = i % 7;
    b[i] = -(int64_t)(i % 5) - 1;
    sumA += a[i];
    sumB += b[i];
  }
  auto inA = accl.Allocate1D<int64_t>(a);
  auto inB = accl.Allocate1D<int64_t>(b);
  auto outA = accl.Allocate1D<int64_t>(1);
  auto outB = accl.Allocate1D<int64_t>(1);
  auto s1 = accl.CreateStream();
  auto s2 = accl.CreateStream();
  for (int round = 0; round < 20; ++round) {
    reduce(*s1, inA->View(), outA->View());
    reduce(*s2, inB->View(), outB->View());
    reduce(*s1, inA->View(), outA->View());
    reduce(*s2, inB->View(), outB->View());
  }
  s1->Synchronize();
  s2->Synchronize();
  CHECK(outA->GetAsArray1D()[0] == sumA);
  CHECK(outB->GetAsArray1D()[0] == sumB);
  // the cached delegate behind Reduce(accelerator, stream, input, output)
  Reduce<int64_t, SRO::AddInt64>(accl, *s1, inA->View(), outB->View());
  Reduce<int64_t, SRO::AddInt64>(accl, *s2, inB->View(), outA->View());
  s1->Synchronize();
  s2->Synchronize();
  CHECK(outB->GetAsArray1D()[0] == sumA);
  CHECK(outA->GetAsArray1D()[0] == sumB);
  // ReduceAsync (ReductionExtensions.cs:230-236): two tasks at once, one per stream
  auto futureA = ReduceAsync<int64_t, SRO::AddInt64>(accl, *s1, inA->View());
  auto futureB = ReduceAsync<int64_t, SRO::AddInt64>(accl, *s2, inB->View());
  CHECK(futureA.get() == sumA);
  CHECK(futureB.get() == sumB);
}

// Floating-point bins (the launchers exist for every AtomicNumericType,
// HistogramLaunchers.tt:25-34): counts below 2^24 are exact in a float bin, a bin
// near 2^24 stops there, and a bin that holds MaxValue reports overflow
// (HistogramOperations.tt:36-40).
template <typename T, typename TBin> void HistogramFloatBinTests(Accelerator& accl) {
  using Modulo = HistogramOperations::ModuloBinOperation;
  const int length = 1024, numBins = 64;
  std::vector<T> input((size_t)length);
  for (int i = 0; i < length; ++i) input[i] = (T)(i + 1);
  std::vector<TBin> start((size_t)numBins), expected((size_t)numBins);
  for (int b = 0; b < numBins; ++b) {
    start[b] = (TBin)(0.5 * b);
    expected[b] = (TBin)(0.5 * b + length / numBins);
  }
  start[3] = (TBin)16777210.0;  // 16 more: a float bin stops at 2^24
  expected[3] = sizeof(TBin) == 4 ? (TBin)16777216.0 : (TBin)16777226.0;
  auto dIn = accl.Allocate1D<T>(input);
  auto hist = accl.Allocate1D<TBin>(start);
  auto overflow = accl.Allocate1D<int32_t>(1);
  overflow->MemSetToZero();
  Histogram<T, Stride1D::Dense, Modulo, TBin>(accl, accl.DefaultStream(), dIn->View(),
                                              hist->View(), overflow->View());
  accl.Synchronize();
  CHECK(Verify(hist->GetAsArray1D(), expected));
  CHECK(overflow->GetAsArray1D()[0] == 0);
  auto full = accl.Allocate1D<TBin>(std::vector<TBin>{std::numeric_limits<TBin>::max()});
  Histogram<T, Stride1D::Dense, Modulo, TBin>(accl, accl.DefaultStream(), dIn->View(),
                                              full->View(), overflow->View());
  accl.Synchronize();
  CHECK(full->GetAsArray1D()[0] == std::numeric_limits<TBin>::max());
  CHECK(overflow->GetAsArray1D()[0] == 1);
}

// ---- HistogramTests -----------------------------------------------------------
template <typename T, typename TBin> void HistogramTests(Accelerator& accl) {
  using Modulo = HistogramOperations::ModuloBinOperation;
  for (int numBins : {64, 256}) {  // Histogram_CreateBin...(64|256, 1024) (:99-144)
    const int length = 1024;
    std::vector<T> input((size_t)length);
    for (int i = 0; i < length; ++i) input[i] = (T)(i + 1);
    std::vector<TBin> expected((size_t)numBins, 0);
    for (T v : input) {
      long bin;
      if (std::is_floating_point<T>::value) bin = (long)std::fabs(std::fmod((double)v, (double)numBins));
      else bin = std::labs((long)((long long)v % numBins));
      expected[(size_t)bin] += 1;
    }
    auto dIn = accl.Allocate1D<T>(input);
    auto hist = accl.Allocate1D<TBin>(numBins);
    hist->MemSetToZero();
    auto overflow = accl.Allocate1D<int32_t>(1);
    overflow->MemSetToZero();
    accl.Synchronize();
    Histogram<T, Stride1D::Dense, Modulo, TBin>(accl, accl.DefaultStream(), dIn->View(),
                                                hist->View(), overflow->View());
    accl.Synchronize();
    CHECK(Verify(hist->GetAsArray1D(), expected));
    CHECK(overflow->GetAsArray1D()[0] == 0);
  }
  {  // HistogramOverflow_CreateBin... (:146-203)
    const int length = 32;
    std::vector<T> input((size_t)length);
    for (int i = 0; i < length; ++i) input[i] = (T)(i + 1);
    const TBin start = (TBin)(std::numeric_limits<TBin>::max() - (TBin)length - 1);
    auto dIn = accl.Allocate1D<T>(input);
    auto hist = accl.Allocate1D<TBin>(std::vector<TBin>{start});
    auto overflow = accl.Allocate1D<int32_t>(1);
    overflow->MemSetToZero();
    using Unsigned = typename std::make_unsigned<TBin>::type;
    Histogram<T, Stride1D::Dense, Modulo, TBin>(accl, accl.DefaultStream(), dIn->View(),
                                                hist->View(), overflow->View());
    accl.Synchronize();
    CHECK(hist->GetAsArray1D()[0] == (TBin)((Unsigned)start + (Unsigned)length));
    CHECK(overflow->GetAsArray1D()[0] == 0);
    Histogram<T, Stride1D::Dense, Modulo, TBin>(accl, accl.DefaultStream(), dIn->View(),
                                                hist->View(), overflow->View());
    accl.Synchronize();
    CHECK(hist->GetAsArray1D()[0] == (TBin)((Unsigned)start + (Unsigned)(2 * length)));
    CHECK(overflow->GetAsArray1D()[0] == 1);
  }
}

// ---- TempViewManagerTests (host only) ------------------------------------------
template <typename T> void TempViewManagerTests() {
  int32_t* fake = reinterpret_cast<int32_t*>(0x10000);  // never dereferenced
  const int64_t rel = ((int64_t)sizeof(T) + 3) / 4;
  {  // AlignedAllocation (TempViewManagerTests.cs:51-63)
    TempViewManager m(ArrayView<int32_t>(fake, rel * 2), "buffer");
    m.Allocate<T>(1);
    m.Allocate<T>(1);
    CHECK(m.NumInts() == rel * 2);
  }
  if (sizeof(T) > sizeof(int32_t)) {  // UnalignedAllocation (:65-84)
    TempViewManager m(ArrayView<int32_t>(fake, rel + 1), "buffer");
    m.Allocate<uint8_t>(1);
    EXPECT_THROW(m.Allocate<T>(1), InvalidOperationException);
  }
  {
    TempViewManager m(ArrayView<int32_t>(fake, rel), "buffer");
    m.Allocate<T>(1);
    EXPECT_THROW(m.Allocate<T>(1), ArgumentOutOfRangeException);
  }
  EXPECT_THROW(TempViewManager(ArrayView<int32_t>(), "temp"), ArgumentNullException);
}

int main(int argc, char** argv) {
  const bool hostOnly = argc > 1 && std::string(argv[1]) == "--host";
  RUN(TempViewManagerTests<int8_t>());
  RUN(TempViewManagerTests<int32_t>());
  RUN(TempViewManagerTests<int64_t>());
  RUN(TempViewManagerTests<double>());
  if (!hostOnly) {
    Accelerator accl(0);
    RUN((RadixTests<int32_t, RSO::AscendingInt32, RSO::DescendingInt32>(accl)));
    RUN((RadixTests<int64_t, RSO::AscendingInt64, RSO::DescendingInt64>(accl)));
    RUN((RadixTests<uint32_t, RSO::AscendingUInt32, RSO::DescendingUInt32>(accl)));
    RUN((RadixTests<uint64_t, RSO::AscendingUInt64, RSO::DescendingUInt64>(accl)));
    RUN((RadixTests<float, RSO::AscendingFloat, RSO::DescendingFloat>(accl)));
    RUN((RadixTests<double, RSO::AscendingDouble, RSO::DescendingDouble>(accl)));
    RUN(RadixSortSequencerPairs(accl));
    RUN(RadixSortStrided(accl));
    RUN(RadixSortErrors(accl));
    RUN((ScanTests<int32_t, SRO::AddInt32>(accl, 1027)));
    RUN((ScanTests<int32_t, SRO::MaxInt32>(accl, 1027)));
    RUN((ScanTests<int64_t, SRO::MinInt64>(accl, 1027)));
    RUN((ScanTests<uint32_t, SRO::AddUInt32>(accl, 1027)));
    RUN((ScanTests<uint64_t, SRO::MaxUInt64>(accl, 1027)));
    RUN((ScanTests<float, SRO::AddFloat>(accl, 1000)));
    RUN((ScanTests<double, SRO::MinDouble>(accl, 1000)));
    RUN(ScanErrors(accl));
    RUN((ReduceTests<int32_t, SRO::AddInt32>(accl, 1027)));
    RUN((ReduceTests<int64_t, SRO::MaxInt64>(accl, 1027)));
    RUN((ReduceTests<uint32_t, SRO::MinUInt32>(accl, 1027)));
    RUN((ReduceTests<uint64_t, SRO::AddUInt64>(accl, 1027)));
    RUN((ReduceTests<float, SRO::AddFloat>(accl, 1000)));
    RUN((ReduceTests<double, SRO::MaxDouble>(accl, 1000)));
    RUN(ReduceErrors(accl));
    RUN(ReduceOnTwoStreams(accl));
    RUN((HistogramTests<int32_t, int32_t>(accl)));
    RUN((HistogramTests<uint8_t, uint32_t>(accl)));
    RUN((HistogramTests<int64_t, int64_t>(accl)));
    RUN((HistogramTests<float, uint64_t>(accl)));
    RUN((HistogramTests<int16_t, int32_t>(accl)));
    RUN((HistogramFloatBinTests<int32_t, float>(accl)));
    RUN((HistogramFloatBinTests<float, double>(accl)));
    RUN(UniqueTests<int32_t>(accl));
    RUN(UniqueTests<uint8_t>(accl));
    RUN(UniqueTests<int64_t>(accl));
    RUN(UniqueTests<float>(accl));
    RUN(UniqueTests<double>(accl));
    RUN(UniqueErrors(accl));
    RUN((SequencerTests<int32_t, ilgpu::Sequencers::IndexSequencer>(accl)));
    RUN((SequencerTests<int8_t, ilgpu::Sequencers::Int8Sequencer>(accl)));
    RUN((SequencerTests<uint64_t, ilgpu::Sequencers::UInt64Sequencer>(accl)));
    RUN((SequencerTests<double, ilgpu::Sequencers::DoubleSequencer>(accl)));
    RUN(InitializeAndReorderTests<int32_t>(accl));
    RUN(InitializeAndReorderTests<uint16_t>(accl));
    RUN(InitializeAndReorderTests<double>(accl));
    RUN(TransformTests(accl));
    RUN(CastFromIndexTests<int32_t>(accl));
    RUN(CastFromIndexTests<int64_t>(accl));
    RUN(CastFromIndexTests<uint32_t>(accl));
    RUN(CastFromIndexTests<uint64_t>(accl));
    RUN(CastFromIndexTests<float>(accl));
    RUN(CastFromIndexTests<double>(accl));
    RUN(ReorderTransformTests<int32_t>(accl));
    RUN(ReorderTransformTests<uint64_t>(accl));
    RUN(ReorderTransformTests<float>(accl));
  }
  std::printf("%d test groups, %d failed checks\n", g_run, g_failed);
  return g_failed == 0 ? 0 : 1;
}
