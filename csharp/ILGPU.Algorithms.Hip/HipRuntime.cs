// What ILGPU lacks for a HIP device: ILGPU has no HIP accelerator
// (AcceleratorType is CPU, Velocity, Cuda, OpenCL: Src/ILGPU/Runtime/Accelerator.cs:26-47)
// and Accelerator cannot be subclassed without a Backend (Accelerator.cs:198).
// The three classes below supply device memory and streams so that the
// reference's ArrayView/ArrayView1D types can point at HIP memory:
//   HipMemoryBuffer  derives from MemoryBuffer (its constructor is protected,
//                    MemoryBuffer.cs:35) with no owning accelerator; NativePtr
//                    is the hipMalloc pointer, which is all that
//                    ArrayView.LoadEffectiveAddressAsPtr needs
//                    (ArrayView.cs:465-478);
//   HipStream        derives from AcceleratorStream (AcceleratorStream.cs:37);
//   HipAccelerator   the object the extension methods hang off, with the
//                    members the samples use (Allocate1D, CreateStream,
//                    DefaultStream, Synchronize).
using System;
using System.Runtime.InteropServices;
using ILGPU.Runtime;

namespace ILGPU.Algorithms.Hip
{
    internal static unsafe class HipRuntimeNativeMethods
    {
        private const string LibName = "libamdhip64.so";
        internal const int MemcpyHostToDevice = 1, MemcpyDeviceToHost = 2, MemcpyDeviceToDevice = 3;

        [DllImport(LibName)] internal static extern int hipSetDevice(int device);
        [DllImport(LibName)] internal static extern int hipDeviceSynchronize();
        [DllImport(LibName)] internal static extern int hipMalloc(out IntPtr ptr, UIntPtr bytes);
        [DllImport(LibName)] internal static extern int hipFree(IntPtr ptr);
        [DllImport(LibName)] internal static extern int hipMemcpy(
            void* dst, void* src, UIntPtr bytes, int kind);
        [DllImport(LibName)] internal static extern int hipMemcpyAsync(
            void* dst, void* src, UIntPtr bytes, int kind, IntPtr stream);
        [DllImport(LibName)] internal static extern int hipMemsetAsync(
            void* dst, int value, UIntPtr bytes, IntPtr stream);
        [DllImport(LibName)] internal static extern int hipStreamCreate(out IntPtr stream);
        [DllImport(LibName)] internal static extern int hipStreamDestroy(IntPtr stream);
        [DllImport(LibName)] internal static extern int hipStreamSynchronize(IntPtr stream);
        [DllImport(LibName)] internal static extern IntPtr hipGetErrorString(int error);

        internal static void Check(int error)
        {
            if (error != 0)
                throw new HipAlgorithmsException(
                    HipAlgorithmsStatus.Runtime, error,
                    Marshal.PtrToStringAnsi(hipGetErrorString(error)) ?? "HIP error");
        }
    }

    /// <summary>A HIP stream behind ILGPU's AcceleratorStream type.</summary>
    public sealed class HipStream : AcceleratorStream
    {
        private readonly bool owned;

        internal HipStream(IntPtr stream, bool owned) : base(null)
        {
            StreamPtr = stream;
            this.owned = owned;
        }

        /// <summary>The hipStream_t (the analogue of CudaStream.StreamPtr).</summary>
        public IntPtr StreamPtr { get; private set; }

        public override void Synchronize() =>
            HipRuntimeNativeMethods.Check(HipRuntimeNativeMethods.hipStreamSynchronize(StreamPtr));

        protected override ProfilingMarker AddProfilingMarkerInternal() =>
            throw new NotSupportedException("profiling markers: use HipAccelerator.EnableKernelProfiling");

        protected override void DisposeAcceleratorObject(bool disposing)
        {
            if (owned && StreamPtr != IntPtr.Zero)
                HipRuntimeNativeMethods.hipStreamDestroy(StreamPtr);
            StreamPtr = IntPtr.Zero;
        }

        /// <summary>The native stream of any stream handed to this layer.</summary>
        internal static IntPtr PtrOf(AcceleratorStream stream) =>
            stream is HipStream hip
            ? hip.StreamPtr
            : throw new NotSupportedException("the stream is not a HipStream");
    }

    /// <summary>hipMalloc memory behind ILGPU's MemoryBuffer type.</summary>
    public unsafe class HipMemoryBuffer : MemoryBuffer
    {
        internal HipMemoryBuffer(long length, int elementSize) : base(null, length, elementSize)
        {
            HipRuntimeNativeMethods.Check(HipRuntimeNativeMethods.hipMalloc(
                out IntPtr ptr, new UIntPtr((ulong)(length * elementSize))));
            NativePtr = ptr;
        }

        protected override void MemSet(
            AcceleratorStream stream, byte value, in ArrayView<byte> targetView) =>
            HipRuntimeNativeMethods.Check(HipRuntimeNativeMethods.hipMemsetAsync(
                targetView.LoadEffectiveAddressAsPtr().ToPointer(), value,
                new UIntPtr((ulong)targetView.LengthInBytes), HipStream.PtrOf(stream)));

        protected override void CopyTo(
            AcceleratorStream stream, in ArrayView<byte> sourceView,
            in ArrayView<byte> targetView) =>
            Copy(stream, sourceView, targetView);

        protected override void CopyFrom(
            AcceleratorStream stream, in ArrayView<byte> sourceView,
            in ArrayView<byte> targetView) =>
            Copy(stream, sourceView, targetView);

        private static void Copy(
            AcceleratorStream stream, in ArrayView<byte> source, in ArrayView<byte> target)
        {
            bool sourceOnDevice = source.Buffer is HipMemoryBuffer;
            bool targetOnDevice = target.Buffer is HipMemoryBuffer;
            int kind = sourceOnDevice
                ? (targetOnDevice ? HipRuntimeNativeMethods.MemcpyDeviceToDevice
                                  : HipRuntimeNativeMethods.MemcpyDeviceToHost)
                : HipRuntimeNativeMethods.MemcpyHostToDevice;
            HipRuntimeNativeMethods.Check(HipRuntimeNativeMethods.hipMemcpyAsync(
                target.LoadEffectiveAddressAsPtr().ToPointer(),
                source.LoadEffectiveAddressAsPtr().ToPointer(),
                new UIntPtr((ulong)source.LengthInBytes), kind, HipStream.PtrOf(stream)));
        }

        protected override void DisposeAcceleratorObject(bool disposing)
        {
            if (NativePtr != IntPtr.Zero)
                HipRuntimeNativeMethods.hipFree(NativePtr);
            NativePtr = IntPtr.Zero;
        }
    }

    /// <summary>A typed one-dimensional buffer (MemoryBuffer1D of the reference).</summary>
    public sealed unsafe class HipMemoryBuffer1D<T> : HipMemoryBuffer where T : unmanaged
    {
        internal HipMemoryBuffer1D(long length) : base(length, sizeof(T)) { }

        /// <summary>The whole buffer as a dense view.</summary>
        public ArrayView<T> View => new ArrayView<T>(this, 0, Length);

        public void CopyFromCPU(T[] data)
        {
            if (data.LongLength > Length) throw new ArgumentOutOfRangeException(nameof(data));
            fixed (T* p = data)
                HipRuntimeNativeMethods.Check(HipRuntimeNativeMethods.hipMemcpy(
                    NativePtr.ToPointer(), p, new UIntPtr((ulong)(data.LongLength * sizeof(T))),
                    HipRuntimeNativeMethods.MemcpyHostToDevice));
        }

        public T[] GetAsArray1D()
        {
            var result = new T[Length];
            fixed (T* p = result)
                HipRuntimeNativeMethods.Check(HipRuntimeNativeMethods.hipMemcpy(
                    p, NativePtr.ToPointer(), new UIntPtr((ulong)(Length * sizeof(T))),
                    HipRuntimeNativeMethods.MemcpyDeviceToHost));
            return result;
        }

        public void MemSetToZero(AcceleratorStream stream) =>
            MemSet(stream, 0, 0, LengthInBytes);
    }

    /// <summary>One HIP device: what the extension methods of this layer extend.</summary>
    public sealed class HipAccelerator : IDisposable
    {
        public HipAccelerator(int device = 0)
        {
            Device = device;
            HipRuntimeNativeMethods.Check(HipRuntimeNativeMethods.hipSetDevice(device));
            DefaultStream = new HipStream(IntPtr.Zero, owned: false);
            // The sort ranks keys with returning LDS atomics and needs their lanes
            // served in lane order; the library asks every device once.  Asked
            // here, the answer is there before any sort (also one on a stream
            // that is being captured, which could not wait for it), and a device
            // that fails is refused at construction (NotSupportedException).
            HipAlgorithmsException.ThrowIfFailed(
                HipAlgorithmsNativeMethods.ilgpu_hip_sort_check_device(IntPtr.Zero));
        }

        public int Device { get; }

        /// <summary>The device's default (null) stream.</summary>
        public HipStream DefaultStream { get; }

        public HipStream CreateStream()
        {
            HipRuntimeNativeMethods.Check(HipRuntimeNativeMethods.hipStreamCreate(out IntPtr s));
            return new HipStream(s, owned: true);
        }

        public HipMemoryBuffer1D<T> Allocate1D<T>(long length) where T : unmanaged =>
            new HipMemoryBuffer1D<T>(length);

        public HipMemoryBuffer1D<T> Allocate1D<T>(T[] data) where T : unmanaged
        {
            var buffer = new HipMemoryBuffer1D<T>(data.LongLength);
            buffer.CopyFromCPU(data);
            return buffer;
        }

        public void Synchronize() =>
            HipRuntimeNativeMethods.Check(HipRuntimeNativeMethods.hipDeviceSynchronize());

        /// <summary>Version of the native library (major * 100 + minor).</summary>
        public static int NativeLibraryVersion => HipAlgorithmsNativeMethods.ilgpu_hip_version();

        /// <summary>Switches the library's per-kernel timing on or off (the counterpart
        /// of ILGPU's ProfilingMarker, ProfilingMarker.cs:19-61): while it is on, every
        /// kernel launch of the library is bracketed by a pair of HIP events on its
        /// stream.  Process-wide; off by default.</summary>
        public static void EnableKernelProfiling(bool enabled) =>
            HipAlgorithmsException.ThrowIfFailed(
                HipAlgorithmsNativeMethods.ilgpu_hip_profile_enable(enabled ? 1 : 0));

        /// <summary>Launches and total milliseconds recorded for one kernel name
        /// ("sort_onesweep", "scan", "reduce_partials", "histogram", ...) since the
        /// last query of that name; waits for the recorded events.</summary>
        public static (long Launches, double TotalMilliseconds) QueryKernelProfile(
            string kernelName)
        {
            HipAlgorithmsException.ThrowIfFailed(
                HipAlgorithmsNativeMethods.ilgpu_hip_profile_query(
                    kernelName, out long launches, out double totalMs),
                nameof(kernelName));
            return (launches, totalMs);
        }

        public void Dispose() => DefaultStream.Dispose();
    }
}
