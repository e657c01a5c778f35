// Host layer above the C ABI, mirroring the C# surface of ILGPU.Algorithms for
// the radix sort / scan / reduce / histogram path: same names, argument order,
// validation and exception kinds, so that code written against the reference
// (accelerator.CreateRadixSort<T, TStride, TOp>() ... sort(stream, view, temp))
// reads the same here.  Header only; link with libilgpu_hip_algorithms.so and
// the HIP runtime.
//
//   reference                                         here
//   ILGPU.Runtime.Accelerator / AcceleratorStream     ilgpu::Accelerator / AcceleratorStream (HIP device, hipStream_t)
//   MemoryBuffer1D<T, Stride1D.Dense>                 ilgpu::MemoryBuffer1D<T>
//   ArrayView<T>, ArrayView1D<T, TStride>             ilgpu::ArrayView<T>, ilgpu::ArrayView1D<T, TStride>
//   RadixSortOperations.AscendingInt32 ...            ilgpu::RadixSortOperations::AscendingInt32 ...
//   ScanReduceOperations.AddInt32 ...                 ilgpu::ScanReduceOperations::AddInt32 ...
//   RadixSortExtensions / ScanExtensions /            free functions in ilgpu::Algorithms taking the
//   ReductionExtensions / HistogramExtensions         accelerator as first argument (C# extension methods)
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <functional>
#include <future>
#include <limits>
#include <map>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <typeindex>
#include <typeinfo>
#include <vector>

#include "../../include/ilgpu_hip_algorithms.h"

namespace ilgpu {

// ---- exceptions (System.* kinds the reference throws) ----------------------
struct ArgumentNullException : std::invalid_argument {
  explicit ArgumentNullException(const std::string& p) : std::invalid_argument(p) {}
};
struct ArgumentOutOfRangeException : std::out_of_range {
  explicit ArgumentOutOfRangeException(const std::string& p) : std::out_of_range(p) {}
};
struct NotSupportedException : std::logic_error {
  explicit NotSupportedException(const std::string& m) : std::logic_error(m) {}
};
struct InvalidOperationException : std::logic_error {
  explicit InvalidOperationException(const std::string& m) : std::logic_error(m) {}
};
// Counterpart of CuBlasException (Runtime/Cuda/CuBlasException.cs:98-103).
struct HipAlgorithmsException : std::runtime_error {
  int32_t status;
  HipAlgorithmsException(int32_t s, const std::string& m)
      : std::runtime_error(m), status(s) {}
  static void ThrowIfFailed(int32_t status, const char* param = "") {
    switch (status) {
      case ILGPU_HIP_SUCCESS: return;
      case ILGPU_HIP_ERROR_NULL_VIEW: throw ArgumentNullException(param);
      case ILGPU_HIP_ERROR_OUT_OF_RANGE: throw ArgumentOutOfRangeException(param);
      case ILGPU_HIP_ERROR_NOT_SUPPORTED:
        throw NotSupportedException(ilgpu_hip_status_string(status));
      case ILGPU_HIP_ERROR_UNALIGNED_TEMP:
        throw InvalidOperationException(ilgpu_hip_status_string(status));
      default:
        throw HipAlgorithmsException(
            status, std::string(ilgpu_hip_status_string(status)) + " (hipError " +
                        std::to_string(ilgpu_hip_last_runtime_error()) + ")");
    }
  }
};

inline void CheckHip(hipError_t e) {
  if (e != hipSuccess)
    throw HipAlgorithmsException(ILGPU_HIP_ERROR_RUNTIME, hipGetErrorString(e));
}

using Index1D = int32_t;
using LongIndex1D = int64_t;

// ---- element type codes -----------------------------------------------------
template <typename T> struct TypeCode;
#define ILGPU_TYPE_CODE(T, C) \
  template <> struct TypeCode<T> { static constexpr int32_t value = C; }
ILGPU_TYPE_CODE(int8_t, ILGPU_HIP_I8);   ILGPU_TYPE_CODE(int16_t, ILGPU_HIP_I16);
ILGPU_TYPE_CODE(int32_t, ILGPU_HIP_I32); ILGPU_TYPE_CODE(int64_t, ILGPU_HIP_I64);
ILGPU_TYPE_CODE(uint8_t, ILGPU_HIP_U8);  ILGPU_TYPE_CODE(uint16_t, ILGPU_HIP_U16);
ILGPU_TYPE_CODE(uint32_t, ILGPU_HIP_U32); ILGPU_TYPE_CODE(uint64_t, ILGPU_HIP_U64);
ILGPU_TYPE_CODE(float, ILGPU_HIP_F32);   ILGPU_TYPE_CODE(double, ILGPU_HIP_F64);
#undef ILGPU_TYPE_CODE
// IEEE binary16 carried as raw bits (System.Half / ILGPU.Half).
struct Half { uint16_t bits; };
template <> struct TypeCode<Half> { static constexpr int32_t value = ILGPU_HIP_F16; };

// ---- strides and views -------------------------------------------------------
namespace Stride1D {
struct Dense { static constexpr int64_t StrideExtent = 1; int64_t Stride() const { return 1; } };
struct General {
  int64_t stride = 1;
  int64_t Stride() const { return stride; }
};
}  // namespace Stride1D

// ArrayView<T> (ArrayView.cs:172-265): a window into device memory.
template <typename T> class ArrayView {
 public:
  ArrayView() = default;
  ArrayView(T* ptr, int64_t length) : ptr_(ptr), length_(length) {}
  // IsValid => Buffer != null && Length > 0 (ArrayView.cs:261-265)
  bool IsValid() const { return ptr_ != nullptr && length_ > 0; }
  int64_t Length() const { return length_; }
  Index1D IntLength() const { return static_cast<Index1D>(length_); }
  T* LoadEffectiveAddressAsPtr() const { return ptr_; }
  ArrayView<T> SubView(int64_t index, int64_t length) const {
    if (index < 0 || length < 0 || index + length > length_)
      throw ArgumentOutOfRangeException("index");
    return ArrayView<T>(ptr_ + index, length);
  }
  ArrayView<T> SubView(int64_t index) const { return SubView(index, length_ - index); }
  template <typename U> ArrayView<U> Cast() const {
    return ArrayView<U>(reinterpret_cast<U*>(ptr_),
                        length_ * (int64_t)sizeof(T) / (int64_t)sizeof(U));
  }
 private:
  T* ptr_ = nullptr;
  int64_t length_ = 0;
};

// ArrayView1D<T, TStride> (Runtime/ArrayViews.tt:114-230).
template <typename T, typename TStride = Stride1D::Dense> class ArrayView1D {
 public:
  ArrayView1D() = default;
  ArrayView1D(ArrayView<T> base, int64_t extent, TStride stride = TStride())
      : base_(base), extent_(extent), stride_(stride) {}
  /* implicit */ ArrayView1D(ArrayView<T> base)
      : base_(base), extent_(base.Length()) {}
  bool IsValid() const { return base_.IsValid(); }
  int64_t Length() const { return extent_; }
  Index1D IntLength() const { return static_cast<Index1D>(extent_); }
  Index1D IntExtent() const { return static_cast<Index1D>(extent_); }
  TStride Stride() const { return stride_; }
  ArrayView<T> BaseView() const { return base_; }
  T* LoadEffectiveAddressAsPtr() const { return base_.LoadEffectiveAddressAsPtr(); }
  ArrayView1D<T, Stride1D::General> AsGeneral() const {
    return ArrayView1D<T, Stride1D::General>(base_, extent_,
                                              Stride1D::General{stride_.Stride()});
  }
 private:
  ArrayView<T> base_;
  int64_t extent_ = 0;
  TStride stride_{};
};

// ---- accelerator, stream, buffers ---------------------------------------------
class AcceleratorStream {
 public:
  explicit AcceleratorStream(hipStream_t s, bool owned) : stream_(s), owned_(owned) {}
  ~AcceleratorStream() { if (owned_) (void)hipStreamDestroy(stream_); }
  AcceleratorStream(const AcceleratorStream&) = delete;
  AcceleratorStream& operator=(const AcceleratorStream&) = delete;
  void Synchronize() { CheckHip(hipStreamSynchronize(stream_)); }
  hipStream_t StreamPtr() const { return stream_; }
 private:
  hipStream_t stream_;
  bool owned_;
};

class Accelerator;

template <typename T> class MemoryBuffer1D {
 public:
  MemoryBuffer1D(int64_t length) : length_(length) {
    if (length < 1) throw ArgumentOutOfRangeException("length");
    CheckHip(hipMalloc(reinterpret_cast<void**>(&ptr_), (size_t)length * sizeof(T)));
  }
  ~MemoryBuffer1D() { (void)hipFree(ptr_); }
  MemoryBuffer1D(const MemoryBuffer1D&) = delete;
  MemoryBuffer1D& operator=(const MemoryBuffer1D&) = delete;
  ArrayView<T> View() const { return ArrayView<T>(ptr_, length_); }
  int64_t Length() const { return length_; }
  void MemSetToZero() { CheckHip(hipMemset(ptr_, 0, (size_t)length_ * sizeof(T))); }
  void CopyFromCPU(AcceleratorStream& stream, const std::vector<T>& data) {
    if ((int64_t)data.size() > length_) throw ArgumentOutOfRangeException("data");
    CheckHip(hipMemcpyAsync(ptr_, data.data(), data.size() * sizeof(T),
                            hipMemcpyHostToDevice, stream.StreamPtr()));
    stream.Synchronize();
  }
  void CopyFromCPU(const std::vector<T>& data) {
    if ((int64_t)data.size() > length_) throw ArgumentOutOfRangeException("data");
    CheckHip(hipMemcpy(ptr_, data.data(), data.size() * sizeof(T), hipMemcpyHostToDevice));
  }
  std::vector<T> GetAsArray1D() const {
    std::vector<T> out((size_t)length_);
    CheckHip(hipMemcpy(out.data(), ptr_, (size_t)length_ * sizeof(T), hipMemcpyDeviceToHost));
    return out;
  }
 private:
  T* ptr_ = nullptr;
  int64_t length_;
};

// The HIP device the algorithms run on (stands where ILGPU's Accelerator does).
class Accelerator {
 public:
  explicit Accelerator(int device = 0) : device_(device), default_(nullptr, false) {
    CheckHip(hipSetDevice(device));
    // The sort needs the lanes of an LDS atomic served in lane order; the
    // library asks every device once.  Asked here, the answer is there before
    // any sort, and a device that fails is refused (NotSupportedException).
    HipAlgorithmsException::ThrowIfFailed(ilgpu_hip_sort_check_device(nullptr));
  }
  AcceleratorStream& DefaultStream() { return default_; }
  std::unique_ptr<AcceleratorStream> CreateStream() {
    hipStream_t s;
    CheckHip(hipStreamCreate(&s));
    return std::unique_ptr<AcceleratorStream>(new AcceleratorStream(s, true));
  }
  template <typename T> std::unique_ptr<MemoryBuffer1D<T>> Allocate1D(int64_t length) {
    return std::unique_ptr<MemoryBuffer1D<T>>(new MemoryBuffer1D<T>(length));
  }
  template <typename T>
  std::unique_ptr<MemoryBuffer1D<T>> Allocate1D(const std::vector<T>& data) {
    auto b = Allocate1D<T>((int64_t)data.size());
    b->CopyFromCPU(data);
    return b;
  }
  void Synchronize() { CheckHip(hipDeviceSynchronize()); }
  int Device() const { return device_; }
  // Objects the algorithms keep per accelerator (cached delegates and their
  // scratch), created on first use and released with the accelerator, the way
  // ILGPU caches loaded kernels per accelerator.
  template <typename TKey, typename TObject>
  std::shared_ptr<TObject> GetOrCreateCached(const std::function<std::shared_ptr<TObject>()>& make) {
    std::lock_guard<std::mutex> lock(cache_mutex_);
    std::shared_ptr<void>& slot = cache_[std::type_index(typeid(TKey))];
    if (!slot) slot = make();
    return std::static_pointer_cast<TObject>(slot);
  }
 private:
  int device_;
  AcceleratorStream default_;
  std::mutex cache_mutex_;
  std::map<std::type_index, std::shared_ptr<void>> cache_;
};

// ---- functors ------------------------------------------------------------------
// IRadixSortOperation<T> (IRadixSortOperation.cs:18-38): only the built-in
// Ascending*/Descending* structs of RadixSortOperations.tt:30-125 exist natively.
namespace RadixSortOperations {
template <typename T, bool DESC> struct Operation {
  using Type = T;
  static constexpr bool Descending = DESC;
  static constexpr int NumBits = (int)sizeof(T) * 8;
};
#define ILGPU_SORT_OP(Name, T)                      \
  using Ascending##Name = Operation<T, false>;      \
  using Descending##Name = Operation<T, true>
ILGPU_SORT_OP(Int8, int8_t);   ILGPU_SORT_OP(Int16, int16_t);
ILGPU_SORT_OP(Int32, int32_t); ILGPU_SORT_OP(Int64, int64_t);
ILGPU_SORT_OP(UInt8, uint8_t); ILGPU_SORT_OP(UInt16, uint16_t);
ILGPU_SORT_OP(UInt32, uint32_t); ILGPU_SORT_OP(UInt64, uint64_t);
ILGPU_SORT_OP(Half, Half);     ILGPU_SORT_OP(Float, float);
ILGPU_SORT_OP(Double, double);
#undef ILGPU_SORT_OP
}  // namespace RadixSortOperations

// IScanReduceOperation<T> (IScanReduceOperation.cs:18-48), ScanReduceOperations.tt:20-72.
namespace ScanReduceOperations {
template <typename T, int OP> struct Operation {
  using Type = T;
  static constexpr int32_t Op = OP;
  static T Identity() {
    if (OP == ILGPU_HIP_OP_ADD) return T(0);
    if (OP == ILGPU_HIP_OP_MAX) return std::numeric_limits<T>::lowest();
    return std::numeric_limits<T>::max();
  }
};
#define ILGPU_SCAN_OPS(Name, T)                                \
  using Add##Name = Operation<T, ILGPU_HIP_OP_ADD>;            \
  using Max##Name = Operation<T, ILGPU_HIP_OP_MAX>;            \
  using Min##Name = Operation<T, ILGPU_HIP_OP_MIN>
ILGPU_SCAN_OPS(Int32, int32_t); ILGPU_SCAN_OPS(Int64, int64_t);
ILGPU_SCAN_OPS(UInt32, uint32_t); ILGPU_SCAN_OPS(UInt64, uint64_t);
ILGPU_SCAN_OPS(Float, float); ILGPU_SCAN_OPS(Double, double);
#undef ILGPU_SCAN_OPS
}  // namespace ScanReduceOperations

// ScanKind (ScanExtensions.cs:27-38).
enum class ScanKind { Inclusive = ILGPU_HIP_SCAN_INCLUSIVE, Exclusive = ILGPU_HIP_SCAN_EXCLUSIVE };

// Bin locators offered natively (IComputeSingleBinOperation is user code in
// the reference): identity and the modulo locator of HistogramTests.tt:83-94.
namespace HistogramOperations {
struct IdentityBinOperation { static constexpr int32_t Locator = ILGPU_HIP_LOCATOR_IDENTITY; };
struct ModuloBinOperation { static constexpr int32_t Locator = ILGPU_HIP_LOCATOR_MODULO; };
}  // namespace HistogramOperations

// Sequencers for the key/value sort (Sequencers.tt:25-37, Sequencer.cs:36-45).
namespace Sequencers {
template <typename T> struct IndexValueSequencer { using Type = T; };
using IndexSequencer = IndexValueSequencer<int32_t>;
using Int32Sequencer = IndexValueSequencer<int32_t>;
using Int64Sequencer = IndexValueSequencer<int64_t>;
using UInt32Sequencer = IndexValueSequencer<uint32_t>;
using UInt64Sequencer = IndexValueSequencer<uint64_t>;
using Int8Sequencer = IndexValueSequencer<int8_t>;
using Int16Sequencer = IndexValueSequencer<int16_t>;
using UInt8Sequencer = IndexValueSequencer<uint8_t>;
using UInt16Sequencer = IndexValueSequencer<uint16_t>;
using FloatSequencer = IndexValueSequencer<float>;
using DoubleSequencer = IndexValueSequencer<double>;
}  // namespace Sequencers

// Comparison<T> (ComparisonOperations.tt:30-45): CompareTo.
namespace ComparisonOperations {
template <typename T> struct Comparison { using Type = T; };
using ComparisonInt8 = Comparison<int8_t>;     using ComparisonInt16 = Comparison<int16_t>;
using ComparisonInt32 = Comparison<int32_t>;   using ComparisonInt64 = Comparison<int64_t>;
using ComparisonUInt8 = Comparison<uint8_t>;   using ComparisonUInt16 = Comparison<uint16_t>;
using ComparisonUInt32 = Comparison<uint32_t>; using ComparisonUInt64 = Comparison<uint64_t>;
using ComparisonHalf = Comparison<Half>;       using ComparisonFloat = Comparison<float>;
using ComparisonDouble = Comparison<double>;
}  // namespace ComparisonOperations

namespace Algorithms {

// ---- TempViewManager (TempViewManager.cs:23-115) -----------------------------
class TempViewManager {
 public:
  TempViewManager(ArrayView<int32_t> tempView, const std::string& paramName)
      : temp_(tempView), param_(paramName) {
    if (!tempView.IsValid()) throw ArgumentNullException(paramName);
  }
  int64_t NumInts() const { return num_ints_; }
  ArrayView<int32_t> TempView() const { return temp_; }
  template <typename T> ArrayView<T> Allocate(int64_t length) {
    if (length < 1) throw ArgumentOutOfRangeException("numSecondElements");
    const int64_t viewLength = ((int64_t)sizeof(T) * length + 3) / 4;
    if (num_ints_ + viewLength > temp_.Length()) throw ArgumentOutOfRangeException(param_);
    if (std::is_arithmetic<T>::value) {
      const int64_t byteOffset = num_ints_ * 4;
      if (sizeof(T) > 4 && byteOffset % (int64_t)sizeof(T) != 0)
        throw InvalidOperationException("unaligned temp allocation");
    }
    auto sub = temp_.SubView(num_ints_, viewLength);
    num_ints_ += viewLength;
    return sub.template Cast<T>().SubView(0, length);
  }
 private:
  ArrayView<int32_t> temp_;
  std::string param_;
  int64_t num_ints_ = 0;
};

inline Index1D BytesToInts(int64_t bytes) {
  const int64_t ints = (bytes + 3) / 4;
  if (ints > std::numeric_limits<Index1D>::max())
    throw NotSupportedException("temp storage exceeds the 32-bit index range");
  return (Index1D)ints;
}

// ---- radix sort (RadixSortExtensions.cs) ---------------------------------------
template <typename T, typename TStride>
using RadixSort = std::function<void(AcceleratorStream&, ArrayView1D<T, TStride>, ArrayView<int32_t>)>;
template <typename TKey, typename TKeyStride, typename TValue, typename TValueStride>
using RadixSortPairs = std::function<void(AcceleratorStream&, ArrayView1D<TKey, TKeyStride>,
                                          ArrayView1D<TValue, TValueStride>, ArrayView<int32_t>)>;
template <typename T, typename TStride>
using BufferedRadixSort = std::function<void(AcceleratorStream&, ArrayView1D<T, TStride>)>;
template <typename TKey, typename TKeyStride, typename TValue, typename TValueStride>
using BufferedRadixSortPairs = std::function<void(AcceleratorStream&, ArrayView1D<TKey, TKeyStride>,
                                                  ArrayView1D<TValue, TValueStride>)>;

// ComputeRadixSortTempStorageSize (RadixSortExtensions.cs:419-447), in 32-bit ints.
template <typename T, typename TRadixSortOperation>
Index1D ComputeRadixSortTempStorageSize(Accelerator&, Index1D dataLength) {
  int64_t bytes = 0;
  HipAlgorithmsException::ThrowIfFailed(
      ilgpu_hip_radix_sort_temp_bytes(dataLength, TypeCode<T>::value, 0, &bytes), "dataLength");
  return BytesToInts(bytes);
}
// The same for a Stride1D.General view with an element stride above one: the
// sort stages a dense copy of the view in the temp.  The reference has no such
// overload (its kernels index through the view); passing the dense size for a
// strided view throws ArgumentOutOfRangeException("tempView").
template <typename T, typename TRadixSortOperation>
Index1D ComputeRadixSortTempStorageSize(Accelerator&, Index1D dataLength, int64_t stride) {
  int64_t bytes = 0;
  HipAlgorithmsException::ThrowIfFailed(
      ilgpu_hip_radix_sort_temp_bytes_strided(dataLength, TypeCode<T>::value, 0, stride, 1,
                                              &bytes), "dataLength");
  return BytesToInts(bytes);
}
template <typename TKey, typename TValue, typename TRadixSortOperation>
Index1D ComputeRadixSortPairsTempStorageSize(Accelerator&, Index1D dataLength,
                                             int64_t keyStride, int64_t valueStride) {
  int64_t bytes = 0;
  HipAlgorithmsException::ThrowIfFailed(
      ilgpu_hip_radix_sort_temp_bytes_strided(dataLength, TypeCode<TKey>::value,
                                              (int32_t)sizeof(TValue), keyStride,
                                              valueStride, &bytes), "dataLength");
  return BytesToInts(bytes);
}
// ComputeRadixSortPairsTempStorageSize (:384-404); sized in 64-bit bytes first.
template <typename TKey, typename TValue, typename TRadixSortOperation>
Index1D ComputeRadixSortPairsTempStorageSize(Accelerator&, Index1D dataLength) {
  int64_t bytes = 0;
  HipAlgorithmsException::ThrowIfFailed(
      ilgpu_hip_radix_sort_temp_bytes(dataLength, TypeCode<TKey>::value,
                                      (int32_t)sizeof(TValue), &bytes), "dataLength");
  return BytesToInts(bytes);
}

// CreateRadixSort (:1130-1337).
template <typename T, typename TStride, typename TRadixSortOperation>
RadixSort<T, TStride> CreateRadixSort(Accelerator&) {
  static_assert(std::is_same<typename TRadixSortOperation::Type, T>::value,
                "radix sort operation and element type differ");
  if (TRadixSortOperation::NumBits < 1 || TRadixSortOperation::NumBits % 8 != 0)
    throw NotSupportedException("NotSupportedNumberOfRadixSortBits");
  return [](AcceleratorStream& stream, ArrayView1D<T, TStride> input,
            ArrayView<int32_t> tempView) {
    if (!input.IsValid()) throw ArgumentNullException("input");
    if (input.Length() > std::numeric_limits<int32_t>::max())
      throw NotSupportedException("NotSupportedArrayView64");
    TempViewManager viewManager(tempView, "tempView");
    HipAlgorithmsException::ThrowIfFailed(
        ilgpu_hip_radix_sort_keys(
            stream.StreamPtr(), input.LoadEffectiveAddressAsPtr(), input.Length(),
            input.Stride().Stride(), TypeCode<T>::value,
            TRadixSortOperation::Descending ? ILGPU_HIP_SORT_DESCENDING : 0,
            tempView.LoadEffectiveAddressAsPtr(), tempView.Length() * 4),
        "tempView");
  };
}

// CreateRadixSortPairs with a values view (:1084-1118).
template <typename TKey, typename TKeyStride, typename TValue, typename TValueStride,
          typename TRadixSortOperation>
RadixSortPairs<TKey, TKeyStride, TValue, TValueStride> CreateRadixSortPairs(Accelerator&) {
  static_assert(std::is_same<typename TRadixSortOperation::Type, TKey>::value,
                "radix sort operation and key type differ");
  return [](AcceleratorStream& stream, ArrayView1D<TKey, TKeyStride> keys,
            ArrayView1D<TValue, TValueStride> values, ArrayView<int32_t> tempView) {
    if (!keys.IsValid()) throw ArgumentNullException("keys");
    if (!values.IsValid()) throw ArgumentNullException("values");
    if (keys.Length() != values.Length()) throw ArgumentOutOfRangeException("values");
    TempViewManager viewManager(tempView, "tempView");
    HipAlgorithmsException::ThrowIfFailed(
        ilgpu_hip_radix_sort_pairs(
            stream.StreamPtr(), keys.LoadEffectiveAddressAsPtr(), keys.Stride().Stride(),
            values.LoadEffectiveAddressAsPtr(), values.Stride().Stride(), keys.Length(),
            TypeCode<TKey>::value,
            (int32_t)sizeof(TValue),
            TRadixSortOperation::Descending ? ILGPU_HIP_SORT_DESCENDING : 0,
            ILGPU_HIP_VALUES_FROM_VIEW, tempView.LoadEffectiveAddressAsPtr(),
            tempView.Length() * 4),
        "tempView");
  };
}

// CreateRadixSortPairs with a sequencer (:1017-1074): values[i] = (TValue)i.
template <typename TKey, typename TKeyStride, typename TValue, typename TValueStride,
          typename TSequencer, typename TRadixSortOperation>
std::function<void(AcceleratorStream&, ArrayView1D<TKey, TKeyStride>,
                   ArrayView1D<TValue, TValueStride>, TSequencer, ArrayView<int32_t>)>
CreateRadixSortPairsWithSequencer(Accelerator&) {
  static_assert(std::is_same<typename TSequencer::Type, TValue>::value,
                "sequencer and value type differ");
  return [](AcceleratorStream& stream, ArrayView1D<TKey, TKeyStride> keys,
            ArrayView1D<TValue, TValueStride> values, TSequencer,
            ArrayView<int32_t> tempView) {
    if (!keys.IsValid()) throw ArgumentNullException("keys");
    if (!values.IsValid()) throw ArgumentNullException("values");
    if (keys.Length() != values.Length()) throw ArgumentOutOfRangeException("values");
    TempViewManager viewManager(tempView, "tempView");
    HipAlgorithmsException::ThrowIfFailed(
        ilgpu_hip_radix_sort_pairs(
            stream.StreamPtr(), keys.LoadEffectiveAddressAsPtr(), keys.Stride().Stride(),
            values.LoadEffectiveAddressAsPtr(), values.Stride().Stride(), keys.Length(),
            TypeCode<TKey>::value,
            (int32_t)sizeof(TValue),
            TRadixSortOperation::Descending ? ILGPU_HIP_SORT_DESCENDING : 0,
            // Half/Float/DoubleSequencer convert the index, the others truncate it
            std::is_floating_point<TValue>::value ? ILGPU_HIP_VALUES_FROM_INDEX_AS_FLOAT
                                                  : ILGPU_HIP_VALUES_FROM_INDEX,
            tempView.LoadEffectiveAddressAsPtr(),
            tempView.Length() * 4),
        "tempView");
  };
}

// RadixSortProvider (:168-300, :1378-1437): owns one temp buffer.
class RadixSortProvider {
 public:
  RadixSortProvider(Accelerator& accelerator, Index1D tempStorageSize)
      : accelerator_(accelerator) {
    if (tempStorageSize < 1) throw ArgumentOutOfRangeException("tempStorageSize");
    temp_ = accelerator.Allocate1D<int32_t>(tempStorageSize);
  }
  template <typename T, typename TStride, typename TRadixSortOperation>
  BufferedRadixSort<T, TStride> CreateRadixSort() {
    auto sort = Algorithms::CreateRadixSort<T, TStride, TRadixSortOperation>(accelerator_);
    auto temp = temp_->View();
    return [sort, temp](AcceleratorStream& s, ArrayView1D<T, TStride> v) { sort(s, v, temp); };
  }
  template <typename TKey, typename TKeyStride, typename TValue, typename TValueStride,
            typename TRadixSortOperation>
  BufferedRadixSortPairs<TKey, TKeyStride, TValue, TValueStride> CreateRadixSortPairs() {
    auto sort = Algorithms::CreateRadixSortPairs<TKey, TKeyStride, TValue, TValueStride,
                                                 TRadixSortOperation>(accelerator_);
    auto temp = temp_->View();
    return [sort, temp](AcceleratorStream& s, ArrayView1D<TKey, TKeyStride> k,
                        ArrayView1D<TValue, TValueStride> v) { sort(s, k, v, temp); };
  }
 private:
  Accelerator& accelerator_;
  std::unique_ptr<MemoryBuffer1D<int32_t>> temp_;
};
template <typename T, typename TRadixSortOperation>
std::unique_ptr<RadixSortProvider> CreateRadixSortProvider(Accelerator& a, Index1D dataLength) {
  return std::unique_ptr<RadixSortProvider>(new RadixSortProvider(
      a, ComputeRadixSortTempStorageSize<T, TRadixSortOperation>(a, dataLength)));
}
template <typename TKey, typename TValue, typename TRadixSortOperation>
std::unique_ptr<RadixSortProvider> CreateRadixSortPairsProvider(Accelerator& a,
                                                                Index1D dataLength) {
  return std::unique_ptr<RadixSortProvider>(new RadixSortProvider(
      a, ComputeRadixSortPairsTempStorageSize<TKey, TValue, TRadixSortOperation>(a, dataLength)));
}

// ---- scan (ScanExtensions.cs) ----------------------------------------------------
template <typename T, typename TStrideIn, typename TStrideOut>
using Scan = std::function<void(AcceleratorStream&, ArrayView1D<T, TStrideIn>,
                                ArrayView1D<T, TStrideOut>, ArrayView<int32_t>)>;
template <typename T, typename TStrideIn, typename TStrideOut>
using BufferedScan = std::function<void(AcceleratorStream&, ArrayView1D<T, TStrideIn>,
                                        ArrayView1D<T, TStrideOut>)>;

// ComputeScanTempStorageSize (:158-170), in 32-bit ints.
template <typename T>
LongIndex1D ComputeScanTempStorageSize(Accelerator&, LongIndex1D dataLength) {
  int64_t bytes = 0;
  HipAlgorithmsException::ThrowIfFailed(
      ilgpu_hip_scan_temp_bytes(dataLength, TypeCode<T>::value, &bytes), "dataLength");
  return (bytes + 3) / 4;
}

// CreateScan (:930-959); argument checks as in :675-685.
template <typename T, typename TStrideIn, typename TStrideOut, typename TScanOperation>
Scan<T, TStrideIn, TStrideOut> CreateScan(Accelerator&, ScanKind kind) {
  static_assert(std::is_same<typename TScanOperation::Type, T>::value,
                "scan operation and element type differ");
  return [kind](AcceleratorStream& stream, ArrayView1D<T, TStrideIn> input,
                ArrayView1D<T, TStrideOut> output, ArrayView<int32_t> temp) {
    if (!input.IsValid()) throw ArgumentNullException("input");
    if (!output.IsValid()) throw ArgumentNullException("output");
    if (output.Length() < input.Length()) throw ArgumentOutOfRangeException("output");
    if (input.Length() > std::numeric_limits<int32_t>::max())
      throw NotSupportedException("NotSupportedArrayView64");
    TempViewManager viewManager(temp, "temp");
    HipAlgorithmsException::ThrowIfFailed(
        ilgpu_hip_scan(stream.StreamPtr(), input.LoadEffectiveAddressAsPtr(), input.Length(),
                       input.Stride().Stride(), output.LoadEffectiveAddressAsPtr(),
                       output.Length(), output.Stride().Stride(),
                       TypeCode<T>::value, TScanOperation::Op, (int32_t)kind,
                       temp.LoadEffectiveAddressAsPtr(), temp.Length() * 4),
        "temp");
  };
}

// ScanProvider (:84-142, :968-991).
class ScanProvider {
 public:
  ScanProvider(Accelerator& accelerator, LongIndex1D tempStorageSize)
      : accelerator_(accelerator) {
    if (tempStorageSize < 1) throw ArgumentOutOfRangeException("tempStorageSize");
    temp_ = accelerator.Allocate1D<int32_t>(tempStorageSize);
  }
  template <typename T, typename TStrideIn, typename TStrideOut, typename TScanOperation>
  BufferedScan<T, TStrideIn, TStrideOut> CreateScan(ScanKind kind) {
    auto scan = Algorithms::CreateScan<T, TStrideIn, TStrideOut, TScanOperation>(accelerator_, kind);
    auto temp = temp_->View();
    return [scan, temp](AcceleratorStream& s, ArrayView1D<T, TStrideIn> in,
                        ArrayView1D<T, TStrideOut> out) { scan(s, in, out, temp); };
  }
 private:
  Accelerator& accelerator_;
  std::unique_ptr<MemoryBuffer1D<int32_t>> temp_;
};
template <typename T>
std::unique_ptr<ScanProvider> CreateScanProvider(Accelerator& a, LongIndex1D dataLength) {
  return std::unique_ptr<ScanProvider>(
      new ScanProvider(a, ComputeScanTempStorageSize<T>(a, dataLength)));
}

// ---- reduce (ReductionExtensions.cs) ----------------------------------------------
template <typename T, typename TStride>
using Reduction = std::function<void(AcceleratorStream&, ArrayView1D<T, TStride>, ArrayView<T>)>;

// The scratch of the native reduction (partial results of the first kernel),
// one buffer per stream: the reference's delegate has no hidden state and may
// be invoked on several streams at once (ReductionExtensions.cs:135-167), so
// invocations on different streams must not share partials.  A stream's buffer
// is allocated at the first invocation on that stream and kept.
class ReductionScratch {
 public:
  ReductionScratch(Accelerator& accelerator, int64_t ints) : accelerator_(accelerator), ints_(ints) {}
  ArrayView<int32_t> For(AcceleratorStream& stream) {
    std::lock_guard<std::mutex> lock(mutex_);
    std::unique_ptr<MemoryBuffer1D<int32_t>>& slot = by_stream_[stream.StreamPtr()];
    if (!slot) slot = accelerator_.Allocate1D<int32_t>(ints_);
    return slot->View();
  }
 private:
  Accelerator& accelerator_;
  int64_t ints_;
  std::mutex mutex_;
  std::map<hipStream_t, std::unique_ptr<MemoryBuffer1D<int32_t>>> by_stream_;
};

// CreateReduction (:135-167).  The delegate owns the scratch the native
// kernels need (the reference's delegate has no temp argument).
template <typename T, typename TStride, typename TReduction>
Reduction<T, TStride> CreateReduction(Accelerator& accelerator) {
  static_assert(std::is_same<typename TReduction::Type, T>::value,
                "reduction and element type differ");
  int64_t bytes = 0;
  HipAlgorithmsException::ThrowIfFailed(
      ilgpu_hip_reduce_temp_bytes(1, TypeCode<T>::value, &bytes));
  auto scratch_by_stream = std::make_shared<ReductionScratch>(accelerator, BytesToInts(bytes));
  return [scratch_by_stream](AcceleratorStream& stream, ArrayView1D<T, TStride> input,
                             ArrayView<T> output) {
    if (!input.IsValid()) throw ArgumentNullException("input");
    if (input.Length() < 1) throw ArgumentOutOfRangeException("input");
    if (!output.IsValid()) throw ArgumentNullException("output");
    if (output.Length() < 1) throw ArgumentOutOfRangeException("output");
    const ArrayView<int32_t> scratch = scratch_by_stream->For(stream);
    HipAlgorithmsException::ThrowIfFailed(
        ilgpu_hip_reduce(stream.StreamPtr(), input.LoadEffectiveAddressAsPtr(), input.Length(),
                         input.Stride().Stride(),
                         TypeCode<T>::value, TReduction::Op,
                         output.LoadEffectiveAddressAsPtr(), output.Length(),
                         scratch.LoadEffectiveAddressAsPtr(), scratch.Length() * 4),
        "input");
  };
}

// Reduce into a view (:180-190).  The delegate (and with it the scratch) is
// made once per accelerator, element type and functor and reused: the call
// stays stream-ordered and allocates only the first time a stream is seen.
template <typename T, typename TReduction>
void Reduce(Accelerator& accelerator, AcceleratorStream& stream, ArrayView<T> input,
            ArrayView<T> output) {
  using Delegate = Reduction<T, Stride1D::Dense>;
  struct CacheKey {};  // one per instantiation
  auto reduction = accelerator.GetOrCreateCached<CacheKey, Delegate>([&accelerator]() {
    return std::make_shared<Delegate>(
        CreateReduction<T, Stride1D::Dense, TReduction>(accelerator));
  });
  (*reduction)(stream, input, output);
}
// Reduce returning the value (:204-216): synchronises the stream.
template <typename T, typename TReduction>
T Reduce(Accelerator& accelerator, AcceleratorStream& stream, ArrayView<T> input) {
  auto output = accelerator.Allocate1D<T>(1);
  Reduce<T, TReduction>(accelerator, stream, input, output->View());
  stream.Synchronize();
  return output->GetAsArray1D()[0];
}

// ReduceAsync (:230-236, :302-309): Task.Run(() => Reduce(...)).  The stream
// and the accelerator must outlive the future, as they must outlive the task
// in the reference.
template <typename T, typename TReduction>
std::future<T> ReduceAsync(Accelerator& accelerator, AcceleratorStream& stream,
                           ArrayView<T> input) {
  return std::async(std::launch::async, [&accelerator, &stream, input]() {
    CheckHip(hipSetDevice(accelerator.Device()));  // a new thread starts on device 0
    return Reduce<T, TReduction>(accelerator, stream, input);
  });
}

// ---- histogram (HistogramExtensions.cs, HistogramLaunchers.tt) -------------------
template <typename T, typename TStride, typename TBinType>
using HistogramDelegate = std::function<void(AcceleratorStream&, ArrayView1D<T, TStride>,
                                             ArrayView<TBinType>, ArrayView<int32_t>)>;
template <typename T, typename TStride, typename TBinType>
using HistogramUncheckedDelegate =
    std::function<void(AcceleratorStream&, ArrayView1D<T, TStride>, ArrayView<TBinType>)>;

// CreateHistogram (:293-354); checks as in :322-338.
template <typename T, typename TStride, typename TBinType, typename TLocator>
HistogramDelegate<T, TStride, TBinType> CreateHistogram(Accelerator&) {
  return [](AcceleratorStream& stream, ArrayView1D<T, TStride> view,
            ArrayView<TBinType> histogram, ArrayView<int32_t> histogramOverflow) {
    if (!view.IsValid()) throw ArgumentNullException("view");
    if (view.Length() < 1) throw ArgumentOutOfRangeException("view");
    if (!histogram.IsValid()) throw ArgumentNullException("histogram");
    if (histogram.Length() < 1) throw ArgumentOutOfRangeException("histogram");
    if (!histogramOverflow.IsValid()) throw ArgumentNullException("histogramOverflow");
    if (histogramOverflow.Length() < 1) throw ArgumentOutOfRangeException("histogramOverflow");
    if (view.Length() > std::numeric_limits<int32_t>::max() ||
        histogram.Length() > std::numeric_limits<int32_t>::max())
      throw NotSupportedException("NotSupportedArrayView64");
    HipAlgorithmsException::ThrowIfFailed(
        ilgpu_hip_histogram(stream.StreamPtr(), view.LoadEffectiveAddressAsPtr(), view.Length(),
                            view.Stride().Stride(),
                            TypeCode<T>::value, histogram.LoadEffectiveAddressAsPtr(),
                            histogram.Length(), TypeCode<TBinType>::value, TLocator::Locator,
                            histogramOverflow.LoadEffectiveAddressAsPtr()),
        "view");
  };
}
// CreateHistogramUnchecked (:356-420).
template <typename T, typename TStride, typename TBinType, typename TLocator>
HistogramUncheckedDelegate<T, TStride, TBinType> CreateHistogramUnchecked(Accelerator&) {
  return [](AcceleratorStream& stream, ArrayView1D<T, TStride> view,
            ArrayView<TBinType> histogram) {
    if (!view.IsValid()) throw ArgumentNullException("view");
    if (!histogram.IsValid()) throw ArgumentNullException("histogram");
    if (view.Length() > std::numeric_limits<int32_t>::max() ||
        histogram.Length() > std::numeric_limits<int32_t>::max())
      throw NotSupportedException("NotSupportedArrayView64");
    HipAlgorithmsException::ThrowIfFailed(
        ilgpu_hip_histogram(stream.StreamPtr(), view.LoadEffectiveAddressAsPtr(), view.Length(),
                            view.Stride().Stride(),
                            TypeCode<T>::value, histogram.LoadEffectiveAddressAsPtr(),
                            histogram.Length(), TypeCode<TBinType>::value, TLocator::Locator,
                            nullptr),
        "view");
  };
}
// Histogram / HistogramUnchecked launchers (HistogramLaunchers.tt:52-69).
template <typename T, typename TStride, typename TLocator, typename TBinType>
void Histogram(Accelerator& accelerator, AcceleratorStream& stream, ArrayView1D<T, TStride> view,
               ArrayView<TBinType> histogram, ArrayView<int32_t> histogramOverflow) {
  CreateHistogram<T, TStride, TBinType, TLocator>(accelerator)(stream, view, histogram,
                                                               histogramOverflow);
}
template <typename T, typename TStride, typename TLocator, typename TBinType>
void HistogramUnchecked(Accelerator& accelerator, AcceleratorStream& stream,
                        ArrayView1D<T, TStride> view, ArrayView<TBinType> histogram) {
  CreateHistogramUnchecked<T, TStride, TBinType, TLocator>(accelerator)(stream, view, histogram);
}

// ---- unique (UniqueExtensions.cs) ------------------------------------------------
template <typename T>
using UniqueDelegate = std::function<void(AcceleratorStream&, ArrayView<T>, ArrayView<int64_t>,
                                          ArrayView<int32_t>)>;
// ComputeUniqueTempStorageSize (:116-123), in 32-bit ints.
template <typename T>
int64_t ComputeUniqueTempStorageSize(Accelerator&, int64_t dataLength) {
  int64_t bytes = 0;
  HipAlgorithmsException::ThrowIfFailed(
      ilgpu_hip_unique_temp_bytes(dataLength, TypeCode<T>::value, &bytes), "dataLength");
  return (bytes + 3) / 4;
}
// CreateUnique (:133-190).
template <typename T, typename TComparisonOperation>
UniqueDelegate<T> CreateUnique(Accelerator& accelerator) {
  static_assert(std::is_same<typename TComparisonOperation::Type, T>::value,
                "comparison operation and element type differ");
  Accelerator* accl = &accelerator;
  return [accl](AcceleratorStream& stream, ArrayView<T> input, ArrayView<int64_t> output,
                ArrayView<int32_t> temp) {
    if (!input.IsValid()) throw ArgumentNullException("input");
    if (!output.IsValid()) throw ArgumentNullException("output");
    if (!temp.IsValid()) throw ArgumentNullException("temp");
    if (output.Length() < 1) throw ArgumentOutOfRangeException("output");
    if (input.Length() > std::numeric_limits<int32_t>::max())
      throw NotSupportedException("NotSupportedArrayView64");
    if (temp.Length() < ComputeUniqueTempStorageSize<T>(*accl, input.Length()))
      throw ArgumentOutOfRangeException("temp");
    HipAlgorithmsException::ThrowIfFailed(
        ilgpu_hip_unique(stream.StreamPtr(), input.LoadEffectiveAddressAsPtr(), input.Length(),
                         TypeCode<T>::value, output.LoadEffectiveAddressAsPtr(), output.Length(),
                         temp.LoadEffectiveAddressAsPtr(), temp.Length() * 4),
        "temp");
  };
}
// Unique returning the new length (:199-209): allocates its output and temp and
// synchronises the stream.
template <typename T, typename TComparisonOperation>
int64_t Unique(Accelerator& accelerator, AcceleratorStream& stream, ArrayView<T> input) {
  auto output = accelerator.Allocate1D<int64_t>(1);
  auto temp = accelerator.Allocate1D<int32_t>(
      ComputeUniqueTempStorageSize<T>(accelerator, input.Length()));
  CreateUnique<T, TComparisonOperation>(accelerator)(stream, input, output->View(),
                                                     temp->View());
  stream.Synchronize();
  return output->GetAsArray1D()[0];
}

// ---- initialize (InitializeExtensions.cs:116-176) -----------------------------------
template <typename T, typename TStride>
using Initializer = std::function<void(AcceleratorStream&, ArrayView1D<T, TStride>, T)>;
template <typename T, typename TStride>
Initializer<T, TStride> CreateInitializer(Accelerator&) {
  static_assert(sizeof(T) == 1 || sizeof(T) == 2 || sizeof(T) == 4 || sizeof(T) == 8 ||
                    sizeof(T) == 16,
                "element sizes of 1, 2, 4, 8 or 16 bytes");
  return [](AcceleratorStream& stream, ArrayView1D<T, TStride> view, T value) {
    if (!view.IsValid()) throw ArgumentNullException("view");
    if (view.Length() < 1) throw ArgumentOutOfRangeException("view");
    HipAlgorithmsException::ThrowIfFailed(
        ilgpu_hip_initialize(stream.StreamPtr(), view.LoadEffectiveAddressAsPtr(), view.Length(),
                             view.Stride().Stride(), (int32_t)sizeof(T), &value),
        "view");
  };
}
template <typename T>
void Initialize(Accelerator& accelerator, AcceleratorStream& stream, ArrayView<T> view, T value) {
  CreateInitializer<T, Stride1D::Dense>(accelerator)(stream, ArrayView1D<T, Stride1D::Dense>(view),
                                                     value);
}
template <typename T, typename TStride>
void Initialize(Accelerator& accelerator, AcceleratorStream& stream,
                ArrayView1D<T, TStride> view, T value) {
  CreateInitializer<T, TStride>(accelerator)(stream, view, value);
}

// ---- sequence (SequenceExtensions.cs:238-630), identity sequencers -----------------------
namespace detail {
template <typename T, typename TStride, typename TSequencer>
void RunSequencer(AcceleratorStream& stream, ArrayView1D<T, TStride> view,
                  int64_t sequenceLength, int64_t sequenceBatchLength) {
  static_assert(std::is_same<typename TSequencer::Type, T>::value,
                "sequencer and element type differ");
  HipAlgorithmsException::ThrowIfFailed(
      ilgpu_hip_sequence(stream.StreamPtr(), view.LoadEffectiveAddressAsPtr(), view.Length(),
                         view.Stride().Stride(), TypeCode<T>::value, sequenceLength,
                         sequenceBatchLength),
      "view");
}
template <typename TView> void CheckSequenceView(const TView& view) {
  if (!view.IsValid()) throw ArgumentNullException("view");
  if (view.Length() < 1) throw ArgumentOutOfRangeException("view");
}
}  // namespace detail
// Sequence (:513-524): view[i] = sequencer(i).
template <typename T, typename TStride, typename TSequencer>
void Sequence(Accelerator&, AcceleratorStream& stream, ArrayView1D<T, TStride> view, TSequencer) {
  detail::CheckSequenceView(view);
  detail::RunSequencer<T, TStride, TSequencer>(stream, view, view.Length(), 1);
}
// RepeatedSequence (:542-555): view[i] = sequencer(i % sequenceLength).
template <typename T, typename TStride, typename TSequencer>
void RepeatedSequence(Accelerator&, AcceleratorStream& stream, ArrayView1D<T, TStride> view,
                      int64_t sequenceLength, TSequencer) {
  detail::CheckSequenceView(view);
  if (sequenceLength < 1) throw ArgumentOutOfRangeException("sequenceLength");
  detail::RunSequencer<T, TStride, TSequencer>(stream, view, sequenceLength, 1);
}
// BatchedSequence (:573-586): view[i] = sequencer(i / sequenceBatchLength).
template <typename T, typename TStride, typename TSequencer>
void BatchedSequence(Accelerator&, AcceleratorStream& stream, ArrayView1D<T, TStride> view,
                     int64_t sequenceBatchLength, TSequencer) {
  detail::CheckSequenceView(view);
  if (sequenceBatchLength < 1) throw ArgumentOutOfRangeException("sequenceBatchLength");
  detail::RunSequencer<T, TStride, TSequencer>(stream, view, view.Length(), sequenceBatchLength);
}
// RepeatedBatchedSequence (:613-630).
template <typename T, typename TStride, typename TSequencer>
void RepeatedBatchedSequence(Accelerator&, AcceleratorStream& stream,
                             ArrayView1D<T, TStride> view, int64_t sequenceLength,
                             int64_t sequenceBatchLength, TSequencer) {
  detail::CheckSequenceView(view);
  if (sequenceLength < 1) throw ArgumentOutOfRangeException("sequenceLength");
  if (sequenceBatchLength < 1) throw ArgumentOutOfRangeException("sequenceBatchLength");
  detail::RunSequencer<T, TStride, TSequencer>(stream, view, sequenceLength,
                                               sequenceBatchLength);
}

// ---- reorder (ReorderExtensions.cs:194-214): target[i] = source[reorderView[i]] -------------
template <typename T>
void Reorder(Accelerator&, AcceleratorStream& stream, ArrayView<T> source, ArrayView<T> target,
             ArrayView<Index1D> reorderView) {
  if (!source.IsValid()) throw ArgumentNullException("source");
  if (source.Length() < 1) throw ArgumentOutOfRangeException("source");
  if (!reorderView.IsValid()) throw ArgumentNullException("reorderView");
  if (reorderView.Length() < source.Length()) throw ArgumentOutOfRangeException("reorderView");
  if (source.Length() > std::numeric_limits<int32_t>::max())
    throw NotSupportedException("NotSupportedArrayView64");
  if (!target.IsValid()) throw ArgumentNullException("source");  // sic, TransformExtensions.cs:322-323
  if (target.Length() < reorderView.Length()) throw ArgumentOutOfRangeException("target");
  HipAlgorithmsException::ThrowIfFailed(
      ilgpu_hip_reorder(stream.StreamPtr(), source.LoadEffectiveAddressAsPtr(), source.Length(),
                        target.LoadEffectiveAddressAsPtr(), target.Length(),
                        reorderView.LoadEffectiveAddressAsPtr(), reorderView.Length(),
                        (int32_t)sizeof(T)),
      "target");
}

// ---- transform (TransformExtensions.cs:24-55, 73-115, 255-506) -------------------------------
// The reference accepts any struct implementing ITransformer<TSource, TTarget>; this layer
// accepts the transformers below, each of the form (TTarget)op((TSource)value) with op closed
// in the source type.  They cover IdentityTransformer and the transformers of the reference's
// tests (Generic/AlgorithmsTestData.tt:170-252: IntToLong, UIntToULong, IntToNegInt,
// UInt32ToBitCompInt32, UInt64ToBitCompInt64, <T>Mul2, Index1To<T>).
template <typename T>
struct IdentityTransformer {           // TransformExtensions.cs:42-55
  using Source = T; using Target = T;
  static constexpr int32_t Kind = ILGPU_HIP_TRANSFORM_CONVERT;
  int64_t Factor() const { return 0; }
};
template <typename TSource, typename TTarget>
struct ConvertTransformer {            // value => (TTarget)value
  using Source = TSource; using Target = TTarget;
  static constexpr int32_t Kind = ILGPU_HIP_TRANSFORM_CONVERT;
  int64_t Factor() const { return 0; }
};
template <typename TSource, typename TTarget = TSource>
struct NegateTransformer {             // value => (TTarget)(-value)
  using Source = TSource; using Target = TTarget;
  static constexpr int32_t Kind = ILGPU_HIP_TRANSFORM_NEGATE;
  int64_t Factor() const { return 0; }
};
template <typename TSource, typename TTarget = TSource>
struct BitComplementTransformer {      // value => (TTarget)~value
  using Source = TSource; using Target = TTarget;
  static constexpr int32_t Kind = ILGPU_HIP_TRANSFORM_BIT_COMPLEMENT;
  int64_t Factor() const { return 0; }
};
template <typename TSource, typename TTarget = TSource>
struct MultiplyTransformer {           // value => (TTarget)(value * (TSource)factor)
  using Source = TSource; using Target = TTarget;
  static constexpr int32_t Kind = ILGPU_HIP_TRANSFORM_MULTIPLY;
  int64_t factor = 2;
  int64_t Factor() const { return factor; }
};

template <typename TSource, typename TSourceStride, typename TTarget, typename TTargetStride,
          typename TTransformer>
using StridedTransformer = std::function<void(AcceleratorStream&, ArrayView1D<TSource, TSourceStride>,
                                              ArrayView1D<TTarget, TTargetStride>, TTransformer)>;
template <typename TSource, typename TTarget, typename TTransformer>
using Transformer = std::function<void(AcceleratorStream&, ArrayView<TSource>, ArrayView<TTarget>,
                                       TTransformer)>;
template <typename TSource, typename TTarget, typename TTransformer>
using ReorderTransformer = std::function<void(AcceleratorStream&, ArrayView<TSource>,
                                              ArrayView<TTarget>, ArrayView<Index1D>, TTransformer)>;

// CreateTransformer, strided form (TransformExtensions.cs:289-345).
template <typename TSource, typename TSourceStride, typename TTarget, typename TTargetStride,
          typename TTransformer>
StridedTransformer<TSource, TSourceStride, TTarget, TTargetStride, TTransformer>
CreateTransformer(Accelerator&) {
  static_assert(std::is_same<typename TTransformer::Source, TSource>::value &&
                    std::is_same<typename TTransformer::Target, TTarget>::value,
                "the transformer must map TSource to TTarget");
  return [](AcceleratorStream& stream, ArrayView1D<TSource, TSourceStride> source,
            ArrayView1D<TTarget, TTargetStride> target, TTransformer transformer) {
    if (!source.IsValid()) throw ArgumentNullException("source");
    if (source.Length() < 1) throw ArgumentOutOfRangeException("source");
    if (!target.IsValid()) throw ArgumentNullException("source");  // sic, :308-309
    if (target.Length() < source.Length()) throw ArgumentOutOfRangeException("target");
    HipAlgorithmsException::ThrowIfFailed(
        ilgpu_hip_transform(stream.StreamPtr(), source.LoadEffectiveAddressAsPtr(),
                            source.Length(), source.Stride().Stride(),
                            TypeCode<TSource>::value, target.LoadEffectiveAddressAsPtr(),
                            target.Length(), target.Stride().Stride(), TypeCode<TTarget>::value,
                            TTransformer::Kind, transformer.Factor()),
        "target");
  };
}
// CreateTransformer, dense form (:255-270).
template <typename TSource, typename TTarget, typename TTransformer>
Transformer<TSource, TTarget, TTransformer> CreateTransformer(Accelerator& accelerator) {
  auto launcher = CreateTransformer<TSource, Stride1D::Dense, TTarget, Stride1D::Dense,
                                    TTransformer>(accelerator);
  return [launcher](AcceleratorStream& stream, ArrayView<TSource> source,
                    ArrayView<TTarget> target, TTransformer transformer) {
    launcher(stream, ArrayView1D<TSource, Stride1D::Dense>(source),
             ArrayView1D<TTarget, Stride1D::Dense>(target), transformer);
  };
}
// CreateTransformer<T, TTransformer> (:356-361).
template <typename T, typename TTransformer>
Transformer<T, T, TTransformer> CreateTransformer(Accelerator& accelerator) {
  return CreateTransformer<T, T, TTransformer>(accelerator);
}
// Transform, in place (:377-393), source to target (:411-428) and strided (:479-506).
template <typename T, typename TTransformer>
void Transform(Accelerator& accelerator, AcceleratorStream& stream, ArrayView<T> view,
               TTransformer transformer) {
  CreateTransformer<T, T, TTransformer>(accelerator)(stream, view, view, transformer);
}
template <typename TSource, typename TTarget, typename TTransformer>
void Transform(Accelerator& accelerator, AcceleratorStream& stream, ArrayView<TSource> source,
               ArrayView<TTarget> target, TTransformer transformer) {
  CreateTransformer<TSource, TTarget, TTransformer>(accelerator)(stream, source, target,
                                                                 transformer);
}
template <typename TSource, typename TSourceStride, typename TTarget, typename TTargetStride,
          typename TTransformer>
void Transform(Accelerator& accelerator, AcceleratorStream& stream,
               ArrayView1D<TSource, TSourceStride> source,
               ArrayView1D<TTarget, TTargetStride> target, TTransformer transformer) {
  CreateTransformer<TSource, TSourceStride, TTarget, TTargetStride, TTransformer>(accelerator)(
      stream, source, target, transformer);
}

// CreateReorderTransformer (ReorderExtensions.cs:143-182) and ReorderTransform (:232-297).
template <typename TSource, typename TTarget, typename TTransformer>
ReorderTransformer<TSource, TTarget, TTransformer> CreateReorderTransformer(Accelerator&) {
  static_assert(std::is_same<typename TTransformer::Source, TSource>::value &&
                    std::is_same<typename TTransformer::Target, TTarget>::value,
                "the transformer must map TSource to TTarget");
  return [](AcceleratorStream& stream, ArrayView<TSource> source, ArrayView<TTarget> target,
            ArrayView<Index1D> reorderView, TTransformer transformer) {
    if (!source.IsValid()) throw ArgumentNullException("source");
    if (source.Length() < 1) throw ArgumentOutOfRangeException("source");
    if (!reorderView.IsValid()) throw ArgumentNullException("reorderView");
    if (reorderView.Length() < source.Length()) throw ArgumentOutOfRangeException("reorderView");
    if (source.Length() > std::numeric_limits<int32_t>::max())
      throw NotSupportedException("NotSupportedArrayView64");
    if (!target.IsValid()) throw ArgumentNullException("source");  // sic
    if (target.Length() < reorderView.Length()) throw ArgumentOutOfRangeException("target");
    HipAlgorithmsException::ThrowIfFailed(
        ilgpu_hip_reorder_transform(stream.StreamPtr(), source.LoadEffectiveAddressAsPtr(),
                                    source.Length(), TypeCode<TSource>::value,
                                    target.LoadEffectiveAddressAsPtr(), target.Length(),
                                    TypeCode<TTarget>::value,
                                    reorderView.LoadEffectiveAddressAsPtr(),
                                    reorderView.Length(), TTransformer::Kind,
                                    transformer.Factor()),
        "target");
  };
}
template <typename T, typename TTransformer>
void ReorderTransform(Accelerator& accelerator, AcceleratorStream& stream, ArrayView<T> source,
                      ArrayView<T> target, ArrayView<Index1D> reorderView,
                      TTransformer transformer) {
  CreateReorderTransformer<T, T, TTransformer>(accelerator)(stream, source, target, reorderView,
                                                            transformer);
}
template <typename TSource, typename TTarget, typename TTransformer>
void ReorderTransform(Accelerator& accelerator, AcceleratorStream& stream,
                      ArrayView<TSource> source, ArrayView<TTarget> target,
                      ArrayView<Index1D> reorderView, TTransformer transformer) {
  CreateReorderTransformer<TSource, TTarget, TTransformer>(accelerator)(
      stream, source, target, reorderView, transformer);
}

}  // namespace Algorithms
}  // namespace ilgpu
