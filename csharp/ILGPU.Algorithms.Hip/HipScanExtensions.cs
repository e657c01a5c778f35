// CreateScan, ComputeScanTempStorageSize and the scan provider with the
// reference's signatures (ScanExtensions.cs:52-76, 158-170, 84-142, 930-991).
using System;
using ILGPU.Algorithms.ScanReduceOperations;
using ILGPU.Runtime;
using static ILGPU.Algorithms.Hip.HipAlgorithmsNativeMethods;

namespace ILGPU.Algorithms.Hip
{
    public static unsafe class HipScanExtensions
    {
        /// <summary>ComputeScanTempStorageSize (:158-170), in 32-bit integers.</summary>
        public static LongIndex1D ComputeScanTempStorageSize<T>(
            this HipAccelerator accelerator,
            LongIndex1D dataLength)
            where T : unmanaged
        {
            HipAlgorithmsException.ThrowIfFailed(
                ilgpu_hip_scan_temp_bytes(dataLength, HipTypeMap.ElementType<T>(), out long bytes),
                nameof(dataLength));
            return HipTypeMap.BytesToInts(bytes);
        }

        /// <summary>CreateScan (:930-959); argument checks in the order of :675-685.</summary>
        public static Scan<T, TStrideIn, TStrideOut> CreateScan<
            T,
            TStrideIn,
            TStrideOut,
            TScanOperation>(
            this HipAccelerator accelerator,
            ScanKind kind)
            where T : unmanaged
            where TStrideIn : struct, IStride1D
            where TStrideOut : struct, IStride1D
            where TScanOperation : struct, IScanReduceOperation<T>
        {
            var (elementType, op) = HipTypeMap.ScanReduceOperation<T, TScanOperation>();
            int nativeKind = HipTypeMap.Kind(kind);
            return (stream, input, output, temp) =>
            {
                if (!input.IsValid)
                    throw new ArgumentNullException(nameof(input));
                if (!output.IsValid)
                    throw new ArgumentNullException(nameof(output));
                if (output.Extent < input.Extent)
                    throw new ArgumentOutOfRangeException(nameof(output));
                if (input.Extent > int.MaxValue)
                    throw new NotSupportedException("NotSupportedArrayView64");
                if (!temp.IsValid)
                    throw new ArgumentNullException(nameof(temp));
                HipAlgorithmsException.ThrowIfFailed(
                    ilgpu_hip_scan(
                        HipStream.PtrOf(stream),
                        input.BaseView.LoadEffectiveAddressAsPtr().ToPointer(),
                        input.Extent,
                        input.Stride.StrideExtent,
                        output.BaseView.LoadEffectiveAddressAsPtr().ToPointer(),
                        output.Extent,
                        output.Stride.StrideExtent,
                        elementType,
                        op,
                        nativeKind,
                        temp.LoadEffectiveAddressAsPtr().ToPointer(),
                        temp.Length * sizeof(int)),
                    nameof(temp));
            };
        }

        /// <summary>The scan on the library's own scratch (ilgpu_hip_scan_static): no
        /// temp view and no allocation, at most 1 GiB of input, one call at a time
        /// per device.  No counterpart in the reference.</summary>
        public static BufferedScan<T, TStrideIn, TStrideOut> CreateScanWithoutTemp<
            T,
            TStrideIn,
            TStrideOut,
            TScanOperation>(
            this HipAccelerator accelerator,
            ScanKind kind)
            where T : unmanaged
            where TStrideIn : struct, IStride1D
            where TStrideOut : struct, IStride1D
            where TScanOperation : struct, IScanReduceOperation<T>
        {
            var (elementType, op) = HipTypeMap.ScanReduceOperation<T, TScanOperation>();
            int nativeKind = HipTypeMap.Kind(kind);
            return (stream, input, output) =>
            {
                if (!input.IsValid)
                    throw new ArgumentNullException(nameof(input));
                if (!output.IsValid)
                    throw new ArgumentNullException(nameof(output));
                HipAlgorithmsException.ThrowIfFailed(
                    ilgpu_hip_scan_static(
                        HipStream.PtrOf(stream),
                        input.BaseView.LoadEffectiveAddressAsPtr().ToPointer(),
                        input.Extent,
                        input.Stride.StrideExtent,
                        output.BaseView.LoadEffectiveAddressAsPtr().ToPointer(),
                        output.Extent,
                        output.Stride.StrideExtent,
                        elementType,
                        op,
                        nativeKind),
                    nameof(output));
            };
        }

        /// <summary>CreateScanProvider(dataLength in ints) (:968-973).</summary>
        public static HipScanProvider CreateScanProvider(
            this HipAccelerator accelerator,
            LongIndex1D dataLength) =>
            dataLength < 1
            ? throw new ArgumentOutOfRangeException(nameof(dataLength))
            : new HipScanProvider(accelerator, dataLength);

        /// <summary>CreateScanProvider for elements of type T (:984-991).</summary>
        public static HipScanProvider CreateScanProvider<T>(
            this HipAccelerator accelerator,
            LongIndex1D dataLength)
            where T : unmanaged =>
            accelerator.CreateScanProvider(
                accelerator.ComputeScanTempStorageSize<T>(dataLength));
    }

    /// <summary>ScanProvider (ScanExtensions.cs:84-142).</summary>
    public sealed class HipScanProvider : IDisposable
    {
        private readonly HipAccelerator accelerator;
        private readonly HipMemoryBuffer1D<int> tempBuffer;

        internal HipScanProvider(HipAccelerator accelerator, LongIndex1D tempSize)
        {
            this.accelerator = accelerator;
            tempBuffer = accelerator.Allocate1D<int>(tempSize);
        }

        public BufferedScan<T, TStrideIn, TStrideOut> CreateScan<
            T, TStrideIn, TStrideOut, TScanOperation>(ScanKind kind)
            where T : unmanaged
            where TStrideIn : struct, IStride1D
            where TStrideOut : struct, IStride1D
            where TScanOperation : struct, IScanReduceOperation<T>
        {
            var scan = accelerator.CreateScan<T, TStrideIn, TStrideOut, TScanOperation>(kind);
            var temp = tempBuffer.View;
            return (stream, input, output) => scan(stream, input, output, temp);
        }

        public void Dispose() => tempBuffer.Dispose();
    }
}
