// CreateRadixSort / CreateRadixSortPairs and their sizing helpers and providers
// with the reference's signatures (RadixSortExtensions.cs:37-160, 384-447,
// 1017-1337, 1378-1437), over libilgpu_hip_algorithms.so.  The delegate types
// (RadixSort<,>, RadixSortPairs<,,,>, Buffered...) and the functor structs are
// the reference's own.
using System;
using ILGPU.Algorithms.RadixSortOperations;
using ILGPU.Algorithms.Sequencers;
using ILGPU.Runtime;
using static ILGPU.Algorithms.Hip.HipAlgorithmsNativeMethods;

namespace ILGPU.Algorithms.Hip
{
    public static unsafe class HipRadixSortExtensions
    {
        private static long ValidLength<T, TStride>(
            ArrayView1D<T, TStride> view, string name)
            where T : unmanaged
            where TStride : struct, IStride1D
        {
            if (!view.IsValid)
                throw new ArgumentNullException(name);
            // RadixSortExtensions.cs:1195-1199
            if (view.Extent > int.MaxValue)
                throw new NotSupportedException("NotSupportedArrayView64");
            return view.Extent;
        }

        private static void CheckTemp(ArrayView<int> temp)
        {
            // TempViewManager.cs:33-41
            if (!temp.IsValid)
                throw new ArgumentNullException(nameof(temp));
        }

        /// <summary>ComputeRadixSortTempStorageSize (RadixSortExtensions.cs:419-447):
        /// the temp size in 32-bit integers.</summary>
        public static Index1D ComputeRadixSortTempStorageSize<T, TRadixSortOperation>(
            this HipAccelerator accelerator,
            Index1D dataLength)
            where T : unmanaged
            where TRadixSortOperation : struct, IRadixSortOperation<T>
        {
            var (keyType, _) = HipTypeMap.SortOperation<T, TRadixSortOperation>();
            HipAlgorithmsException.ThrowIfFailed(
                ilgpu_hip_radix_sort_temp_bytes(dataLength, keyType, 0, out long bytes),
                nameof(dataLength));
            return checked((int)HipTypeMap.BytesToInts(bytes));
        }

        /// <summary>ComputeRadixSortPairsTempStorageSize (:384-403).</summary>
        public static Index1D ComputeRadixSortPairsTempStorageSize<
            TKey,
            TValue,
            TRadixSortOperation>(
            this HipAccelerator accelerator,
            Index1D dataLength)
            where TKey : unmanaged
            where TValue : unmanaged
            where TRadixSortOperation : struct, IRadixSortOperation<TKey>
        {
            var (keyType, _) = HipTypeMap.SortOperation<TKey, TRadixSortOperation>();
            HipAlgorithmsException.ThrowIfFailed(
                ilgpu_hip_radix_sort_temp_bytes(
                    dataLength, keyType, sizeof(TValue), out long bytes),
                nameof(dataLength));
            return checked((int)HipTypeMap.BytesToInts(bytes));
        }

        /// <summary>The temp size, in 32-bit integers, of a sort of views with element
        /// strides above one (the strided views are gathered into a dense copy at
        /// the end of temp, sorted there and scattered back); valueBytes is 0 for
        /// keys only.  The reference's sizing helpers have no stride argument.</summary>
        public static LongIndex1D ComputeRadixSortTempStorageSize<T, TRadixSortOperation>(
            this HipAccelerator accelerator,
            LongIndex1D dataLength,
            int valueBytes,
            long keyStride,
            long valueStride)
            where T : unmanaged
            where TRadixSortOperation : struct, IRadixSortOperation<T>
        {
            var (keyType, _) = HipTypeMap.SortOperation<T, TRadixSortOperation>();
            HipAlgorithmsException.ThrowIfFailed(
                ilgpu_hip_radix_sort_temp_bytes_strided(
                    dataLength, keyType, valueBytes, keyStride, valueStride, out long bytes),
                nameof(dataLength));
            return HipTypeMap.BytesToInts(bytes);
        }

        /// <summary>How many 8-bit passes the last sort that used temp ran and how
        /// many it found unnecessary (a pass whose digit is the same for every key
        /// is skipped); same length, key type and value size (0 for keys only) as
        /// that sort.  Waits for the stream.  The reference runs every pass whatever
        /// the keys and has nothing to report.</summary>
        public static (int Executed, int Skipped) GetRadixSortPasses<T, TRadixSortOperation>(
            this HipAccelerator accelerator,
            AcceleratorStream stream,
            ArrayView<int> temp,
            LongIndex1D dataLength,
            int valueBytes = 0)
            where T : unmanaged
            where TRadixSortOperation : struct, IRadixSortOperation<T>
        {
            var (keyType, _) = HipTypeMap.SortOperation<T, TRadixSortOperation>();
            CheckTemp(temp);
            HipAlgorithmsException.ThrowIfFailed(
                ilgpu_hip_radix_sort_passes(
                    HipStream.PtrOf(stream),
                    temp.LoadEffectiveAddressAsPtr().ToPointer(),
                    temp.Length * sizeof(int),
                    dataLength,
                    keyType,
                    valueBytes,
                    out int executed,
                    out int skipped),
                nameof(temp));
            return (executed, skipped);
        }

        /// <summary>The library's own check of the one hardware property the ranking
        /// of a pass rests on (lanes of one LDS atomic served in lane order), played
        /// over `rows` rows per wave: the number of lanes found out of order, 0 on
        /// gfx950.  Every sort runs a short form of it once per device by itself
        /// (HipAccelerator's constructor asks for it); this is the long form for
        /// diagnostics.</summary>
        public static long CountLdsAtomicOrderViolations(
            this HipAccelerator accelerator,
            AcceleratorStream stream,
            int rows = 256)
        {
            using var mismatches = accelerator.Allocate1D<long>(1);
            HipAlgorithmsException.ThrowIfFailed(
                ilgpu_hip_selftest_lds_atomic_order(
                    HipStream.PtrOf(stream),
                    rows,
                    (long*)mismatches.View.LoadEffectiveAddressAsPtr().ToPointer()),
                nameof(rows));
            stream.Synchronize();
            return mismatches.GetAsArray1D()[0];
        }

        /// <summary>CreateRadixSort (:1130-1337).</summary>
        public static RadixSort<T, TStride> CreateRadixSort<
            T,
            TStride,
            TRadixSortOperation>(
            this HipAccelerator accelerator)
            where T : unmanaged
            where TStride : struct, IStride1D
            where TRadixSortOperation : struct, IRadixSortOperation<T>
        {
            var (keyType, flags) = HipTypeMap.SortOperation<T, TRadixSortOperation>();
            return (stream, view, temp) =>
            {
                long length = ValidLength(view, nameof(view));
                CheckTemp(temp);
                HipAlgorithmsException.ThrowIfFailed(
                    ilgpu_hip_radix_sort_keys(
                        HipStream.PtrOf(stream),
                        view.BaseView.LoadEffectiveAddressAsPtr().ToPointer(),
                        length,
                        view.Stride.StrideExtent,
                        keyType,
                        flags,
                        temp.LoadEffectiveAddressAsPtr().ToPointer(),
                        temp.Length * sizeof(int)),
                    nameof(temp));
            };
        }

        /// <summary>CreateRadixSortPairs with a values view (:1017-1074).</summary>
        public static RadixSortPairs<TKey, TKeyStride, TValue, TValueStride>
            CreateRadixSortPairs<
            TKey,
            TKeyStride,
            TValue,
            TValueStride,
            TRadixSortOperation>(
            this HipAccelerator accelerator)
            where TKey : unmanaged
            where TKeyStride : struct, IStride1D
            where TValue : unmanaged
            where TValueStride : struct, IStride1D
            where TRadixSortOperation : struct, IRadixSortOperation<TKey>
        {
            var (keyType, flags) = HipTypeMap.SortOperation<TKey, TRadixSortOperation>();
            return (stream, keys, values, temp) =>
            {
                long length = ValidLength(keys, nameof(keys));
                if (!values.IsValid)
                    throw new ArgumentNullException(nameof(values));
                // :1053-1054
                if (values.Extent != keys.Extent)
                    throw new ArgumentOutOfRangeException(nameof(values));
                CheckTemp(temp);
                HipAlgorithmsException.ThrowIfFailed(
                    ilgpu_hip_radix_sort_pairs(
                        HipStream.PtrOf(stream),
                        keys.BaseView.LoadEffectiveAddressAsPtr().ToPointer(),
                        keys.Stride.StrideExtent,
                        values.BaseView.LoadEffectiveAddressAsPtr().ToPointer(),
                        values.Stride.StrideExtent,
                        length,
                        keyType,
                        sizeof(TValue),
                        flags,
                        HipTypeMap.ValuesFromView,
                        temp.LoadEffectiveAddressAsPtr().ToPointer(),
                        temp.Length * sizeof(int)),
                    nameof(temp));
            };
        }

        /// <summary>CreateRadixSortPairs with a sequencer (:1076-1118): the
        /// identity sequencers (value = element index) are generated on the
        /// device; other sequencers are not supported.</summary>
        public static RadixSortPairs<TKey, TKeyStride, TValue, TValueStride, TSequencer>
            CreateRadixSortPairs<
            TKey,
            TKeyStride,
            TValue,
            TValueStride,
            TSequencer,
            TRadixSortOperation>(
            this HipAccelerator accelerator)
            where TKey : unmanaged
            where TKeyStride : struct, IStride1D
            where TValue : unmanaged
            where TValueStride : struct, IStride1D
            where TSequencer : struct, ISequencer<TValue>
            where TRadixSortOperation : struct, IRadixSortOperation<TKey>
        {
            var (keyType, flags) = HipTypeMap.SortOperation<TKey, TRadixSortOperation>();
            int valueSource = HipTypeMap.ValueSource<TValue, TSequencer>();
            return (stream, keys, outputValues, sequencer, temp) =>
            {
                long length = ValidLength(keys, nameof(keys));
                if (!outputValues.IsValid)
                    throw new ArgumentNullException(nameof(outputValues));
                if (outputValues.Extent != keys.Extent)
                    throw new ArgumentOutOfRangeException(nameof(outputValues));
                CheckTemp(temp);
                HipAlgorithmsException.ThrowIfFailed(
                    ilgpu_hip_radix_sort_pairs(
                        HipStream.PtrOf(stream),
                        keys.BaseView.LoadEffectiveAddressAsPtr().ToPointer(),
                        keys.Stride.StrideExtent,
                        outputValues.BaseView.LoadEffectiveAddressAsPtr().ToPointer(),
                        outputValues.Stride.StrideExtent,
                        length,
                        keyType,
                        sizeof(TValue),
                        flags,
                        valueSource,
                        temp.LoadEffectiveAddressAsPtr().ToPointer(),
                        temp.Length * sizeof(int)),
                    nameof(temp));
            };
        }

        /// <summary>CreateRadixSortProvider(tempStorageSize) (:1378-1383).</summary>
        public static HipRadixSortProvider CreateRadixSortProvider(
            this HipAccelerator accelerator,
            Index1D tempStorageSize) =>
            tempStorageSize < 1
            ? throw new ArgumentOutOfRangeException(nameof(tempStorageSize))
            : new HipRadixSortProvider(accelerator, tempStorageSize);

        /// <summary>CreateRadixSortProvider for keys of a length (:1396-1406).</summary>
        public static HipRadixSortProvider CreateRadixSortProvider<T, TRadixSortOperation>(
            this HipAccelerator accelerator,
            Index1D dataLength)
            where T : unmanaged
            where TRadixSortOperation : struct, IRadixSortOperation<T> =>
            accelerator.CreateRadixSortProvider(
                accelerator.ComputeRadixSortTempStorageSize<T, TRadixSortOperation>(dataLength));

        /// <summary>CreateRadixSortProvider for pairs of a length (:1422-1437).</summary>
        public static HipRadixSortProvider CreateRadixSortProvider<
            TKey,
            TValue,
            TRadixSortOperation>(
            this HipAccelerator accelerator,
            Index1D dataLength)
            where TKey : unmanaged
            where TValue : unmanaged
            where TRadixSortOperation : struct, IRadixSortOperation<TKey> =>
            accelerator.CreateRadixSortProvider(
                accelerator.ComputeRadixSortPairsTempStorageSize<
                    TKey, TValue, TRadixSortOperation>(dataLength));
    }

    /// <summary>RadixSortProvider (RadixSortExtensions.cs:168-300): owns one temp
    /// buffer and hands out delegates without a temp argument.  Not thread safe,
    /// like the reference's (:167).</summary>
    public sealed class HipRadixSortProvider : IDisposable
    {
        private readonly HipAccelerator accelerator;
        private readonly HipMemoryBuffer1D<int> tempBuffer;

        internal HipRadixSortProvider(HipAccelerator accelerator, Index1D tempSize)
        {
            this.accelerator = accelerator;
            tempBuffer = accelerator.Allocate1D<int>(tempSize);
        }

        public BufferedRadixSort<T, TStride> CreateRadixSort<T, TStride, TRadixSortOperation>()
            where T : unmanaged
            where TStride : struct, IStride1D
            where TRadixSortOperation : struct, IRadixSortOperation<T>
        {
            var sort = accelerator.CreateRadixSort<T, TStride, TRadixSortOperation>();
            var temp = tempBuffer.View;
            return (stream, view) => sort(stream, view, temp);
        }

        public BufferedRadixSortPairs<TKey, TKeyStride, TValue, TValueStride>
            CreateRadixSortPairs<TKey, TKeyStride, TValue, TValueStride, TRadixSortOperation>()
            where TKey : unmanaged
            where TKeyStride : struct, IStride1D
            where TValue : unmanaged
            where TValueStride : struct, IStride1D
            where TRadixSortOperation : struct, IRadixSortOperation<TKey>
        {
            var sort = accelerator.CreateRadixSortPairs<
                TKey, TKeyStride, TValue, TValueStride, TRadixSortOperation>();
            var temp = tempBuffer.View;
            return (stream, keys, values) => sort(stream, keys, values, temp);
        }

        public BufferedRadixSortPairs<TKey, TKeyStride, TValue, TValueStride, TSequencer>
            CreateRadixSortPairs<
            TKey, TKeyStride, TValue, TValueStride, TSequencer, TRadixSortOperation>()
            where TKey : unmanaged
            where TKeyStride : struct, IStride1D
            where TValue : unmanaged
            where TValueStride : struct, IStride1D
            where TSequencer : struct, ISequencer<TValue>
            where TRadixSortOperation : struct, IRadixSortOperation<TKey>
        {
            var sort = accelerator.CreateRadixSortPairs<
                TKey, TKeyStride, TValue, TValueStride, TSequencer, TRadixSortOperation>();
            var temp = tempBuffer.View;
            return (stream, keys, values, sequencer) =>
                sort(stream, keys, values, sequencer, temp);
        }

        public void Dispose() => tempBuffer.Dispose();
    }
}
