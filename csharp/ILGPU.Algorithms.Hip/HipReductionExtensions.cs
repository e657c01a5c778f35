// CreateReduction, Reduce and ReduceAsync with the reference's signatures
// (ReductionExtensions.cs:30-35, 135-309).  The native reduction needs 32 KiB
// of scratch for its partial results; the reference's delegate has no temp
// argument and may run on several streams at once, so the scratch is kept per
// stream inside the delegate.
using System;
using System.Collections.Generic;
using System.Threading.Tasks;
using ILGPU.Algorithms.ScanReduceOperations;
using ILGPU.Runtime;
using static ILGPU.Algorithms.Hip.HipAlgorithmsNativeMethods;

namespace ILGPU.Algorithms.Hip
{
    public static unsafe class HipReductionExtensions
    {
        private sealed class ScratchPerStream
        {
            private readonly HipAccelerator accelerator;
            private readonly long ints;
            private readonly Dictionary<IntPtr, HipMemoryBuffer1D<int>> buffers =
                new Dictionary<IntPtr, HipMemoryBuffer1D<int>>();

            public ScratchPerStream(HipAccelerator accelerator, long ints)
            {
                this.accelerator = accelerator;
                this.ints = ints;
            }

            public ArrayView<int> For(IntPtr stream)
            {
                lock (buffers)
                {
                    if (!buffers.TryGetValue(stream, out var buffer))
                        buffers[stream] = buffer = accelerator.Allocate1D<int>(ints);
                    return buffer.View;
                }
            }
        }

        /// <summary>CreateReduction (:135-167); output[0] is overwritten.</summary>
        public static Reduction<T, TStride> CreateReduction<T, TStride, TReduction>(
            this HipAccelerator accelerator)
            where T : unmanaged
            where TStride : struct, IStride1D
            where TReduction : struct, IScanReduceOperation<T>
        {
            var (elementType, op) = HipTypeMap.ScanReduceOperation<T, TReduction>();
            HipAlgorithmsException.ThrowIfFailed(
                ilgpu_hip_reduce_temp_bytes(1, elementType, out long bytes));
            var scratch = new ScratchPerStream(accelerator, HipTypeMap.BytesToInts(bytes));
            return (stream, input, output) =>
            {
                // :146-153
                if (!input.IsValid)
                    throw new ArgumentNullException(nameof(input));
                if (input.Extent < 1)
                    throw new ArgumentOutOfRangeException(nameof(input));
                if (!output.IsValid)
                    throw new ArgumentNullException(nameof(output));
                if (output.Length < 1)
                    throw new ArgumentOutOfRangeException(nameof(output));
                IntPtr nativeStream = HipStream.PtrOf(stream);
                ArrayView<int> temp = scratch.For(nativeStream);
                HipAlgorithmsException.ThrowIfFailed(
                    ilgpu_hip_reduce(
                        nativeStream,
                        input.BaseView.LoadEffectiveAddressAsPtr().ToPointer(),
                        input.Extent,
                        input.Stride.StrideExtent,
                        elementType,
                        op,
                        output.LoadEffectiveAddressAsPtr().ToPointer(),
                        output.Length,
                        temp.LoadEffectiveAddressAsPtr().ToPointer(),
                        temp.Length * sizeof(int)),
                    nameof(input));
            };
        }

        /// <summary>Reduce into a view (:180-190).</summary>
        public static void Reduce<T, TReduction>(
            this HipAccelerator accelerator,
            AcceleratorStream stream,
            ArrayView<T> input,
            ArrayView<T> output)
            where T : unmanaged
            where TReduction : struct, IScanReduceOperation<T> =>
            accelerator.CreateReduction<T, Stride1D.Dense, TReduction>()(
                stream,
                input,
                output);

        /// <summary>Reduce returning the value (:204-216): waits for the stream.</summary>
        public static T Reduce<T, TReduction>(
            this HipAccelerator accelerator,
            AcceleratorStream stream,
            ArrayView<T> input)
            where T : unmanaged
            where TReduction : struct, IScanReduceOperation<T>
        {
            using var output = accelerator.Allocate1D<T>(1);
            accelerator.Reduce<T, TReduction>(stream, input, output.View);
            stream.Synchronize();
            return output.GetAsArray1D()[0];
        }

        /// <summary>ReduceAsync (:230-236).</summary>
        public static Task<T> ReduceAsync<T, TReduction>(
            this HipAccelerator accelerator,
            AcceleratorStream stream,
            ArrayView<T> input)
            where T : unmanaged
            where TReduction : struct, IScanReduceOperation<T> =>
            Task.Run(() => accelerator.Reduce<T, TReduction>(stream, input));

        /// <summary>Reduce of a strided view into a view (:248-259).</summary>
        public static void Reduce<T, TStride, TReduction>(
            this HipAccelerator accelerator,
            AcceleratorStream stream,
            ArrayView1D<T, TStride> input,
            ArrayView<T> output)
            where T : unmanaged
            where TStride : struct, IStride1D
            where TReduction : struct, IScanReduceOperation<T> =>
            accelerator.CreateReduction<T, TStride, TReduction>()(
                stream,
                input,
                output);

        /// <summary>Reduce of a strided view returning the value (:274-287).</summary>
        public static T Reduce<T, TStride, TReduction>(
            this HipAccelerator accelerator,
            AcceleratorStream stream,
            ArrayView1D<T, TStride> input)
            where T : unmanaged
            where TStride : struct, IStride1D
            where TReduction : struct, IScanReduceOperation<T>
        {
            using var output = accelerator.Allocate1D<T>(1);
            accelerator.Reduce<T, TStride, TReduction>(stream, input, output.View);
            stream.Synchronize();
            return output.GetAsArray1D()[0];
        }

        /// <summary>ReduceAsync of a strided view (:302-309).</summary>
        public static Task<T> ReduceAsync<T, TStride, TReduction>(
            this HipAccelerator accelerator,
            AcceleratorStream stream,
            ArrayView1D<T, TStride> input)
            where T : unmanaged
            where TStride : struct, IStride1D
            where TReduction : struct, IScanReduceOperation<T> =>
            Task.Run(() => accelerator.Reduce<T, TStride, TReduction>(stream, input));
    }
}
