// The C ABI of libilgpu_hip_algorithms.so (include/ilgpu_hip_algorithms.h), one
// DllImport per exported function, in the header's order.  Loading by library
// name follows the reference's native wrappers
// (Src/ILGPU.Algorithms/Runtime/Cuda/API/CuBlasNativeMethods.tt:29-41).
//
// Widths: int32_t = int, int64_t = long, ilgpu_hip_stream_t = IntPtr, every
// device or host pointer = void* / int* / long*, a single-value result pointer
// = out.  tests/test_csharp_binding.py checks every prototype below against the
// header (name, number of arguments, width of each argument).
using System;
using System.Runtime.InteropServices;

namespace ILGPU.Algorithms.Hip
{
    internal static unsafe class HipAlgorithmsNativeMethods
    {
        internal const string LibName = "libilgpu_hip_algorithms.so";

        [DllImport(LibName)] internal static extern int ilgpu_hip_version();
        [DllImport(LibName)] internal static extern IntPtr ilgpu_hip_status_string(int status);
        [DllImport(LibName)] internal static extern int ilgpu_hip_last_runtime_error();
        [DllImport(LibName)] internal static extern int ilgpu_hip_profile_enable(int enabled);
        [DllImport(LibName, CharSet = CharSet.Ansi)]
        internal static extern int ilgpu_hip_profile_query(
            string kernelName, out long launches, out double totalMs);

        [DllImport(LibName)] internal static extern int ilgpu_hip_radix_sort_temp_bytes(
            long n, int keyType, int valueBytes, out long tempBytes);
        [DllImport(LibName)] internal static extern int ilgpu_hip_radix_sort_temp_bytes_strided(
            long n, int keyType, int valueBytes, long keyStride, long valueStride,
            out long tempBytes);
        [DllImport(LibName)] internal static extern int ilgpu_hip_radix_sort_keys(
            IntPtr stream, void* keys, long n, long stride, int keyType, int flags,
            void* temp, long tempBytes);
        [DllImport(LibName)] internal static extern int ilgpu_hip_radix_sort_pairs(
            IntPtr stream, void* keys, long keyStride, void* values, long valueStride, long n,
            int keyType, int valueBytes, int flags, int valueSource, void* temp, long tempBytes);
        [DllImport(LibName)] internal static extern int ilgpu_hip_radix_sort_passes(
            IntPtr stream, void* temp, long tempBytes, long n, int keyType, int valueBytes,
            out int executed, out int skipped);
        [DllImport(LibName)] internal static extern int ilgpu_hip_selftest_lds_atomic_order(
            IntPtr stream, int rows, long* mismatches);
        [DllImport(LibName)] internal static extern int ilgpu_hip_sort_check_device(IntPtr stream);
        [DllImport(LibName)] internal static extern int ilgpu_hip_sort_set_parameter(
            int parameter, int value);

        [DllImport(LibName)] internal static extern int ilgpu_hip_scan_temp_bytes(
            long n, int elemType, out long tempBytes);
        [DllImport(LibName)] internal static extern int ilgpu_hip_scan(
            IntPtr stream, void* input, long inLength, long inStride, void* output,
            long outLength, long outStride, int elemType, int op, int kind, void* temp,
            long tempBytes);
        [DllImport(LibName)] internal static extern int ilgpu_hip_scan_static(
            IntPtr stream, void* input, long inLength, long inStride, void* output,
            long outLength, long outStride, int elemType, int op, int kind);

        [DllImport(LibName)] internal static extern int ilgpu_hip_reduce_temp_bytes(
            long n, int elemType, out long tempBytes);
        [DllImport(LibName)] internal static extern int ilgpu_hip_reduce(
            IntPtr stream, void* input, long n, long stride, int elemType, int op,
            void* output, long outLength, void* temp, long tempBytes);

        [DllImport(LibName)] internal static extern int ilgpu_hip_histogram(
            IntPtr stream, void* input, long n, long stride, int inType, void* bins,
            long numBins, int binType, int locator, int* overflow);

        [DllImport(LibName)] internal static extern int ilgpu_hip_unique_temp_bytes(
            long n, int elemType, out long tempBytes);
        [DllImport(LibName)] internal static extern int ilgpu_hip_unique(
            IntPtr stream, void* input, long n, int elemType, long* newLength,
            long newLengthExtent, void* temp, long tempBytes);

        [DllImport(LibName)] internal static extern int ilgpu_hip_initialize(
            IntPtr stream, void* view, long n, long stride, int elemBytes, void* hostValue);
        [DllImport(LibName)] internal static extern int ilgpu_hip_sequence(
            IntPtr stream, void* view, long n, long stride, int elemType, long sequenceLength,
            long batchLength);
        [DllImport(LibName)] internal static extern int ilgpu_hip_reorder(
            IntPtr stream, void* source, long sourceLength, void* target, long targetLength,
            int* order, long orderLength, int elemBytes);
        [DllImport(LibName)] internal static extern int ilgpu_hip_transform(
            IntPtr stream, void* source, long sourceLength, long sourceStride, int sourceType,
            void* target, long targetLength, long targetStride, int targetType,
            int transformer, long factor);
        [DllImport(LibName)] internal static extern int ilgpu_hip_reorder_transform(
            IntPtr stream, void* source, long sourceLength, int sourceType, void* target,
            long targetLength, int targetType, int* order, long orderLength, int transformer,
            long factor);
    }
}
