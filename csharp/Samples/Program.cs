// The reference's algorithm samples on a HIP device
// (Samples/AlgorithmsRadixSort/Program.cs:59-63, AlgorithmsScan/Program.cs:32-33,
// AlgorithmsReduce/Program.cs:29-31, AlgorithmsHistogram): the same calls with a
// HipAccelerator in place of the ILGPU accelerator.
using System;
using System.Linq;
using ILGPU;
using ILGPU.Algorithms;
using ILGPU.Algorithms.Hip;
using ILGPU.Algorithms.RadixSortOperations;
using ILGPU.Algorithms.ScanReduceOperations;

internal static class Program
{
    private static void Main()
    {
        using var accelerator = new HipAccelerator(0);
        var stream = accelerator.DefaultStream;

        // radix sort: 32 reversed ints
        int[] reversed = Enumerable.Range(0, 32).Reverse().ToArray();
        using (var keys = accelerator.Allocate1D(reversed))
        using (var temp = accelerator.Allocate1D<int>(
            accelerator.ComputeRadixSortTempStorageSize<int, AscendingInt32>(reversed.Length)))
        {
            var sort = accelerator.CreateRadixSort<int, Stride1D.Dense, AscendingInt32>();
            sort(stream, keys.View, temp.View);
            stream.Synchronize();
            Console.WriteLine(string.Join(", ", keys.GetAsArray1D()));
        }

        // inclusive and exclusive scan of 32 twos
        using (var input = accelerator.Allocate1D(Enumerable.Repeat(2, 32).ToArray()))
        using (var output = accelerator.Allocate1D<int>(32))
        using (var provider = accelerator.CreateScanProvider<int>(32))
        {
            foreach (var kind in new[] { ScanKind.Inclusive, ScanKind.Exclusive })
            {
                var scan = provider.CreateScan<int, Stride1D.Dense, Stride1D.Dense, AddInt32>(kind);
                scan(stream, input.View, output.View);
                stream.Synchronize();
                Console.WriteLine(kind + ": " + string.Join(", ", output.GetAsArray1D()));
            }
        }

        // reduce 0..63
        using (var input = accelerator.Allocate1D(Enumerable.Range(0, 64).ToArray()))
        {
            int sum = accelerator.Reduce<int, AddInt32>(stream, input.View);
            Console.WriteLine("sum = " + sum);   // 2016
        }

        // histogram of 1..1024 into 64 bins by value % 64
        using (var input = accelerator.Allocate1D(Enumerable.Range(1, 1024).ToArray()))
        using (var bins = accelerator.Allocate1D<int>(64))
        using (var overflow = accelerator.Allocate1D<int>(1))
        {
            bins.MemSetToZero(stream);
            overflow.MemSetToZero(stream);
            accelerator.Histogram<int, Stride1D.Dense, int, HipModuloBinOperation<int>>(
                stream, input.View, bins.View, overflow.View);
            stream.Synchronize();
            Console.WriteLine("bins: " + string.Join(", ", bins.GetAsArray1D()));   // 16 each
        }
    }
}
