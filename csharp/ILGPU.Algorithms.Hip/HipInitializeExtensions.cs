// CreateInitializer and Initialize with the reference's signatures
// (InitializeExtensions.cs:26-31, 116-176): view[i] = value.
using System;
using ILGPU.Runtime;
using static ILGPU.Algorithms.Hip.HipAlgorithmsNativeMethods;

namespace ILGPU.Algorithms.Hip
{
    public static unsafe class HipInitializeExtensions
    {
        /// <summary>CreateInitializer (:116-136).  Any unmanaged element type of 1, 2,
        /// 4, 8 or 16 bytes (the value is passed as raw bytes).</summary>
        public static Initializer<T, TStride> CreateInitializer<T, TStride>(
            this HipAccelerator accelerator)
            where T : unmanaged
            where TStride : struct, IStride1D
        {
            int elementBytes = sizeof(T);
            if (elementBytes != 1 && elementBytes != 2 && elementBytes != 4 &&
                elementBytes != 8 && elementBytes != 16)
                throw new NotSupportedException($"element type {typeof(T)} of {elementBytes} bytes");
            return (stream, view, value) =>
            {
                if (!view.IsValid)
                    throw new ArgumentNullException(nameof(view));
                if (view.Length < 1)
                    throw new ArgumentOutOfRangeException(nameof(view));
                T local = value;   // the native call copies the bytes before it returns
                HipAlgorithmsException.ThrowIfFailed(
                    ilgpu_hip_initialize(
                        HipStream.PtrOf(stream),
                        view.BaseView.LoadEffectiveAddressAsPtr().ToPointer(),
                        view.Extent,
                        view.Stride.StrideExtent,
                        elementBytes,
                        &local),
                    nameof(view));
            };
        }

        /// <summary>Initialize on a dense view (:146-156).</summary>
        public static void Initialize<T>(
            this HipAccelerator accelerator,
            AcceleratorStream stream,
            ArrayView<T> view,
            T value)
            where T : unmanaged =>
            accelerator.CreateInitializer<T, Stride1D.Dense>()(
                stream,
                view,
                value);

        /// <summary>Initialize on a strided view (:166-176).</summary>
        public static void Initialize<T, TStride>(
            this HipAccelerator accelerator,
            AcceleratorStream stream,
            ArrayView1D<T, TStride> view,
            T value)
            where T : unmanaged
            where TStride : struct, IStride1D =>
            accelerator.CreateInitializer<T, TStride>()(
                stream,
                view,
                value);
    }
}
