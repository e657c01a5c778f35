// Status codes of the C ABI mapped to the exception kinds the reference's
// delegates throw; the typed exception for runtime failures follows
// CuBlasException.ThrowIfFailed (Src/ILGPU.Algorithms/Runtime/Cuda/CuBlasException.cs:98-103).
using System;
using System.Runtime.InteropServices;

namespace ILGPU.Algorithms.Hip
{
    /// <summary>Status codes of ilgpu_hip_status (include/ilgpu_hip_algorithms.h).</summary>
    public enum HipAlgorithmsStatus
    {
        Success = 0,
        NullView = 1,
        OutOfRange = 2,
        NotSupported = 3,
        UnalignedTemp = 4,
        Runtime = 5,
        StaticLimit = 6,
    }

    /// <summary>A HIP runtime call failed inside the native library.</summary>
    [Serializable]
    public sealed class HipAlgorithmsException : Exception
    {
        public HipAlgorithmsException(HipAlgorithmsStatus status, int hipError, string message)
            : base(message)
        {
            Status = status;
            HipError = hipError;
        }

        /// <summary>The status the native call returned.</summary>
        public HipAlgorithmsStatus Status { get; }

        /// <summary>The hipError_t of the failed runtime call.</summary>
        public int HipError { get; }

        internal static string StatusString(int status) =>
            Marshal.PtrToStringAnsi(HipAlgorithmsNativeMethods.ilgpu_hip_status_string(status))
            ?? "unknown status";

        /// <summary>Throws the exception kind that belongs to a non-zero status.</summary>
        /// <param name="status">What the native call returned.</param>
        /// <param name="paramName">The argument the reference would name.</param>
        public static void ThrowIfFailed(int status, string paramName = null)
        {
            switch ((HipAlgorithmsStatus)status)
            {
                case HipAlgorithmsStatus.Success:
                    return;
                case HipAlgorithmsStatus.NullView:
                    throw new ArgumentNullException(paramName ?? "view");
                case HipAlgorithmsStatus.OutOfRange:
                    throw new ArgumentOutOfRangeException(paramName ?? "view");
                case HipAlgorithmsStatus.NotSupported:
                case HipAlgorithmsStatus.StaticLimit:
                    throw new NotSupportedException(StatusString(status));
                case HipAlgorithmsStatus.UnalignedTemp:
                    // TempViewManager.cs:98-106
                    throw new InvalidOperationException(StatusString(status));
                default:
                    throw new HipAlgorithmsException(
                        (HipAlgorithmsStatus)status,
                        HipAlgorithmsNativeMethods.ilgpu_hip_last_runtime_error(),
                        StatusString(status));
            }
        }
    }
}
