// CreateReorderTransformer, Reorder and ReorderTransform with the reference's
// signatures (ReorderExtensions.cs:42-52, 143-297):
//   target[i] = transformer(source[reorderView[i]]).
// The reference wraps the source in a transformer over the index view and runs
// Transform (:152-176); the native library gathers directly.  Transformers are
// the closed set of HipTransformExtensions.cs; Reorder itself is the identity.
using System;
using ILGPU.Runtime;
using static ILGPU.Algorithms.Hip.HipAlgorithmsNativeMethods;

namespace ILGPU.Algorithms.Hip
{
    public static unsafe class HipReorderExtensions
    {
        /// <summary>CreateReorderTransformer (:143-176); argument checks in the
        /// reference's order, then those of the transformer underneath it
        /// (TransformExtensions.cs:304-317: the index view is its source).</summary>
        public static ReorderTransformer<TSource, TTarget, TTransformer>
            CreateReorderTransformer<
            TSource,
            TTarget,
            TTransformer>(
            this HipAccelerator accelerator)
            where TSource : unmanaged
            where TTarget : unmanaged
            where TTransformer : struct, ITransformer<TSource, TTarget>
        {
            int sourceType = HipTypeMap.ElementType<TSource>();
            int targetType = HipTypeMap.ElementType<TTarget>();
            return (stream, source, target, reorderView, transformer) =>
            {
                if (!source.IsValid)
                    throw new ArgumentNullException(nameof(source));
                if (source.Length < 1)
                    throw new ArgumentOutOfRangeException(nameof(source));
                if (!reorderView.IsValid)
                    throw new ArgumentNullException(nameof(reorderView));
                if (reorderView.Length < source.Length)
                    throw new ArgumentOutOfRangeException(nameof(reorderView));
                if (source.Length > int.MaxValue)
                    throw new NotSupportedException("NotSupportedArrayView64");
                if (!target.IsValid)
                    throw new ArgumentNullException(nameof(source));
                if (target.Length < reorderView.Length)
                    throw new ArgumentOutOfRangeException(nameof(target));
                var (code, factor) =
                    HipTypeMap.Transformer<TSource, TTarget, TTransformer>(transformer);
                HipAlgorithmsException.ThrowIfFailed(
                    ilgpu_hip_reorder_transform(
                        HipStream.PtrOf(stream),
                        source.LoadEffectiveAddressAsPtr().ToPointer(),
                        source.Length,
                        sourceType,
                        target.LoadEffectiveAddressAsPtr().ToPointer(),
                        target.Length,
                        targetType,
                        (int*)reorderView.LoadEffectiveAddressAsPtr().ToPointer(),
                        reorderView.Length,
                        code,
                        factor),
                    nameof(reorderView));
            };
        }

        /// <summary>Reorder (:194-207): target[i] = source[reorderView[i]], for any
        /// unmanaged element type of 1, 2, 4, 8 or 16 bytes (the elements are moved
        /// as raw bytes).</summary>
        public static void Reorder<T>(
            this HipAccelerator accelerator,
            AcceleratorStream stream,
            ArrayView<T> source,
            ArrayView<T> target,
            ArrayView<Index1D> reorderView)
            where T : unmanaged
        {
            if (!source.IsValid)
                throw new ArgumentNullException(nameof(source));
            if (source.Length < 1)
                throw new ArgumentOutOfRangeException(nameof(source));
            if (!reorderView.IsValid)
                throw new ArgumentNullException(nameof(reorderView));
            if (reorderView.Length < source.Length)
                throw new ArgumentOutOfRangeException(nameof(reorderView));
            if (source.Length > int.MaxValue)
                throw new NotSupportedException("NotSupportedArrayView64");
            if (!target.IsValid)
                throw new ArgumentNullException(nameof(source));
            if (target.Length < reorderView.Length)
                throw new ArgumentOutOfRangeException(nameof(target));
            HipAlgorithmsException.ThrowIfFailed(
                ilgpu_hip_reorder(
                    HipStream.PtrOf(stream),
                    source.LoadEffectiveAddressAsPtr().ToPointer(),
                    source.Length,
                    target.LoadEffectiveAddressAsPtr().ToPointer(),
                    target.Length,
                    (int*)reorderView.LoadEffectiveAddressAsPtr().ToPointer(),
                    reorderView.Length,
                    sizeof(T)),
                nameof(reorderView));
        }

        /// <summary>ReorderTransform in one element type (:232-249).</summary>
        public static void ReorderTransform<T, TTransformer>(
            this HipAccelerator accelerator,
            AcceleratorStream stream,
            ArrayView<T> source,
            ArrayView<T> target,
            ArrayView<Index1D> reorderView,
            TTransformer transformer)
            where T : unmanaged
            where TTransformer : struct, ITransformer<T, T>
        {
            accelerator.ReorderTransform<T, T, TTransformer>(
                stream,
                source,
                target,
                reorderView,
                transformer);
        }

        /// <summary>ReorderTransform between element types (:275-297).</summary>
        public static void ReorderTransform<TSource, TTarget, TTransformer>(
            this HipAccelerator accelerator,
            AcceleratorStream stream,
            ArrayView<TSource> source,
            ArrayView<TTarget> target,
            ArrayView<Index1D> reorderView,
            TTransformer transformer)
            where TSource : unmanaged
            where TTarget : unmanaged
            where TTransformer : struct, ITransformer<TSource, TTarget>
        {
            accelerator.CreateReorderTransformer<TSource, TTarget, TTransformer>()(
                stream,
                source,
                target,
                reorderView,
                transformer);
        }
    }
}
