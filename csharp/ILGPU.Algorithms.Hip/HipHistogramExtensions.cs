// CreateHistogram / CreateHistogramUnchecked and the Histogram launchers with
// the shape of the reference's single-bin overloads (HistogramExtensions.cs:35-59,
// 293-508; HistogramLaunchers.tt:52-101).  Bin locators are a closed set: the
// two structs below stand for `value` and `|value % numBins|`; the reference
// JIT-compiles arbitrary locator structs, which a native library cannot.
using System;
using ILGPU.Algorithms.HistogramOperations;
using ILGPU.Runtime;
using static ILGPU.Algorithms.Hip.HipAlgorithmsNativeMethods;

namespace ILGPU.Algorithms.Hip
{
    /// <summary>bin = value; values outside [0, numBins) are ignored.</summary>
    public readonly struct HipIdentityBinOperation<T> : IComputeSingleBinOperation<T, Index1D>
        where T : unmanaged
    {
        public Index1D ComputeHistogramBin(T value, Index1D numBins) =>
            throw new NotSupportedException("evaluated on the device by the native library");
    }

    /// <summary>bin = |value % numBins| (the locator of HistogramTests.tt:42-47).</summary>
    public readonly struct HipModuloBinOperation<T> : IComputeSingleBinOperation<T, Index1D>
        where T : unmanaged
    {
        public Index1D ComputeHistogramBin(T value, Index1D numBins) =>
            throw new NotSupportedException("evaluated on the device by the native library");
    }

    public static unsafe class HipHistogramExtensions
    {
        /// <summary>CreateHistogram (:293-354); checks as in :322-338.  The bins
        /// accumulate; histogramOverflow[0] becomes non-zero if a bin passed its
        /// maximum.</summary>
        public static Histogram<T, TStride, TBinType> CreateHistogram<
            T,
            TStride,
            TBinType,
            TLocator>(
            this HipAccelerator accelerator)
            where T : unmanaged
            where TStride : struct, IStride1D
            where TBinType : unmanaged
            where TLocator : struct, IComputeSingleBinOperation<T, Index1D>
        {
            int inType = HipTypeMap.ElementType<T>();
            int binType = HipTypeMap.ElementType<TBinType>();
            int locator = HipTypeMap.Locator<TLocator>();
            return (stream, view, histogram, histogramOverflow) =>
            {
                if (!view.IsValid)
                    throw new ArgumentNullException(nameof(view));
                if (!histogram.IsValid)
                    throw new ArgumentNullException(nameof(histogram));
                if (!histogramOverflow.IsValid)
                    throw new ArgumentNullException(nameof(histogramOverflow));
                if (view.Extent > int.MaxValue || histogram.Length > int.MaxValue)
                    throw new NotSupportedException("NotSupportedArrayView64");
                HipAlgorithmsException.ThrowIfFailed(
                    ilgpu_hip_histogram(
                        HipStream.PtrOf(stream),
                        view.BaseView.LoadEffectiveAddressAsPtr().ToPointer(),
                        view.Extent,
                        view.Stride.StrideExtent,
                        inType,
                        histogram.LoadEffectiveAddressAsPtr().ToPointer(),
                        histogram.Length,
                        binType,
                        locator,
                        (int*)histogramOverflow.LoadEffectiveAddressAsPtr().ToPointer()),
                    nameof(view));
            };
        }

        /// <summary>CreateHistogramUnchecked (:356-420): no overflow view.</summary>
        public static HistogramUnchecked<T, TStride, TBinType> CreateHistogramUnchecked<
            T,
            TStride,
            TBinType,
            TLocator>(
            this HipAccelerator accelerator)
            where T : unmanaged
            where TStride : struct, IStride1D
            where TBinType : unmanaged
            where TLocator : struct, IComputeSingleBinOperation<T, Index1D>
        {
            int inType = HipTypeMap.ElementType<T>();
            int binType = HipTypeMap.ElementType<TBinType>();
            int locator = HipTypeMap.Locator<TLocator>();
            return (stream, view, histogram) =>
            {
                if (!view.IsValid)
                    throw new ArgumentNullException(nameof(view));
                if (!histogram.IsValid)
                    throw new ArgumentNullException(nameof(histogram));
                if (view.Extent > int.MaxValue || histogram.Length > int.MaxValue)
                    throw new NotSupportedException("NotSupportedArrayView64");
                HipAlgorithmsException.ThrowIfFailed(
                    ilgpu_hip_histogram(
                        HipStream.PtrOf(stream),
                        view.BaseView.LoadEffectiveAddressAsPtr().ToPointer(),
                        view.Extent,
                        view.Stride.StrideExtent,
                        inType,
                        histogram.LoadEffectiveAddressAsPtr().ToPointer(),
                        histogram.Length,
                        binType,
                        locator,
                        null),
                    nameof(view));
            };
        }

        /// <summary>Histogram launcher (HistogramLaunchers.tt:52-69).</summary>
        public static void Histogram<T, TStride, TBinType, TLocator>(
            this HipAccelerator accelerator,
            AcceleratorStream stream,
            ArrayView1D<T, TStride> view,
            ArrayView<TBinType> histogram,
            ArrayView<int> histogramOverflow)
            where T : unmanaged
            where TStride : struct, IStride1D
            where TBinType : unmanaged
            where TLocator : struct, IComputeSingleBinOperation<T, Index1D> =>
            accelerator.CreateHistogram<T, TStride, TBinType, TLocator>()(
                stream,
                view,
                histogram,
                histogramOverflow);

        /// <summary>HistogramUnchecked launcher (HistogramLaunchers.tt:71-101).</summary>
        public static void HistogramUnchecked<T, TStride, TBinType, TLocator>(
            this HipAccelerator accelerator,
            AcceleratorStream stream,
            ArrayView1D<T, TStride> view,
            ArrayView<TBinType> histogram)
            where T : unmanaged
            where TStride : struct, IStride1D
            where TBinType : unmanaged
            where TLocator : struct, IComputeSingleBinOperation<T, Index1D> =>
            accelerator.CreateHistogramUnchecked<T, TStride, TBinType, TLocator>()(
                stream,
                view,
                histogram);
    }
}
