// CreateUnique, Unique and ComputeUniqueTempStorageSize with the reference's
// signatures (UniqueExtensions.cs:25-30, 116-209).  The reference removes
// consecutive duplicates group by group, one group at a time
// (SequentialGroupExecutor); the native library does it in one pass with a
// decoupled look-back over the kept counts.  Elements compare as
// first.CompareTo(second) == 0 (ComparisonOperations.tt:26-45): NaNs are equal
// to each other, -0.0 equals +0.0.
using System;
using ILGPU.Runtime;
using static ILGPU.Algorithms.Hip.HipAlgorithmsNativeMethods;

namespace ILGPU.Algorithms.Hip
{
    public static unsafe class HipUniqueExtensions
    {
        /// <summary>ComputeUniqueTempStorageSize (:116-123), in 32-bit integers (the
        /// reference needs one; the look-back needs a status word per tile).</summary>
        public static LongIndex1D ComputeUniqueTempStorageSize<T>(
            this HipAccelerator accelerator,
            LongIndex1D dataLength)
            where T : unmanaged
        {
            HipAlgorithmsException.ThrowIfFailed(
                ilgpu_hip_unique_temp_bytes(dataLength, HipTypeMap.ElementType<T>(), out long bytes),
                nameof(dataLength));
            return HipTypeMap.BytesToInts(bytes);
        }

        /// <summary>CreateUnique (:133-190): the input is compacted in place and the
        /// new length is stored in output[0]; argument checks in the reference's
        /// order.</summary>
        public static Unique<T> CreateUnique<T, TComparisonOperation>(
            this HipAccelerator accelerator)
            where T : unmanaged
            where TComparisonOperation : struct, IComparisonOperation<T>
        {
            int elementType = HipTypeMap.ComparisonOperation<T, TComparisonOperation>();
            return (stream, input, output, temp) =>
            {
                if (!input.IsValid)
                    throw new ArgumentNullException(nameof(input));
                if (!output.IsValid)
                    throw new ArgumentNullException(nameof(output));
                if (!temp.IsValid)
                    throw new ArgumentNullException(nameof(temp));
                if (output.Length < 1)
                    throw new ArgumentOutOfRangeException(nameof(output));
                if (temp.Length < accelerator.ComputeUniqueTempStorageSize<T>(input.Length))
                    throw new ArgumentOutOfRangeException(nameof(temp));
                if (input.Length > int.MaxValue)
                    throw new NotSupportedException("NotSupportedArrayView64");
                HipAlgorithmsException.ThrowIfFailed(
                    ilgpu_hip_unique(
                        HipStream.PtrOf(stream),
                        input.LoadEffectiveAddressAsPtr().ToPointer(),
                        input.Length,
                        elementType,
                        (long*)output.LoadEffectiveAddressAsPtr().ToPointer(),
                        output.Length,
                        temp.LoadEffectiveAddressAsPtr().ToPointer(),
                        temp.Length * sizeof(int)),
                    nameof(temp));
            };
        }

        /// <summary>Unique returning the new length (:199-209): allocates its output
        /// and temp, waits for the stream and reads the length back.</summary>
        public static long Unique<T, TComparisonOperation>(
            this HipAccelerator accelerator,
            AcceleratorStream stream,
            ArrayView<T> input)
            where T : unmanaged
            where TComparisonOperation : struct, IComparisonOperation<T>
        {
            using var output = accelerator.Allocate1D<long>(1);
            using var temp = accelerator.Allocate1D<int>(
                accelerator.ComputeUniqueTempStorageSize<T>(input.Length));
            accelerator.CreateUnique<T, TComparisonOperation>()(
                stream,
                input,
                output.View,
                temp.View);
            stream.Synchronize();
            return output.GetAsArray1D()[0];
        }
    }
}
