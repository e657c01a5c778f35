// typeof(...) look-ups that turn the reference's generic functor arguments into
// the enum codes of the C ABI.  Unknown functors (user-written structs the
// reference would JIT-compile) are NotSupportedException.
using System;
using System.Collections.Generic;
using ILGPU.Algorithms.ComparisonOperations;
using ILGPU.Algorithms.RadixSortOperations;
using ILGPU.Algorithms.ScanReduceOperations;
using ILGPU.Algorithms.Sequencers;

namespace ILGPU.Algorithms.Hip
{
    /// <summary>Codes of include/ilgpu_hip_algorithms.h.</summary>
    public static class HipTypeMap
    {
        // ilgpu_hip_type: NumericTypes of TypeInformation.ttinclude:94-121, in order.
        public const int I8 = 0, I16 = 1, I32 = 2, I64 = 3, U8 = 4, U16 = 5, U32 = 6, U64 = 7,
            F16 = 8, F32 = 9, F64 = 10;
        // ilgpu_hip_op
        public const int OpAdd = 0, OpMax = 1, OpMin = 2;
        // ilgpu_hip_scan_kind: ScanKind.Inclusive / Exclusive (ScanExtensions.cs:27-38)
        public const int ScanInclusive = 0, ScanExclusive = 1;
        // sort flags, value source
        public const int SortDescending = 1, SortFloatTotalOrder = 2;
        public const int ValuesFromView = 0, ValuesFromIndex = 1, ValuesFromIndexAsFloat = 2;
        // ilgpu_hip_transformer
        public const int TransformConvert = 0, TransformNegate = 1, TransformBitComplement = 2,
            TransformMultiply = 3;
        // histogram locators
        public const int LocatorIdentity = 0, LocatorModulo = 1;

        private static readonly Dictionary<Type, int> ElementTypes = new Dictionary<Type, int>
        {
            { typeof(sbyte), I8 }, { typeof(short), I16 }, { typeof(int), I32 },
            { typeof(long), I64 }, { typeof(byte), U8 }, { typeof(ushort), U16 },
            { typeof(uint), U32 }, { typeof(ulong), U64 }, { typeof(Half), F16 },
            { typeof(float), F32 }, { typeof(double), F64 },
            { typeof(Index1D), I32 }, { typeof(LongIndex1D), I64 },
        };

        /// <summary>The element type code of T.</summary>
        public static int ElementType<T>() where T : unmanaged =>
            ElementTypes.TryGetValue(typeof(T), out int code)
            ? code
            : throw new NotSupportedException($"element type {typeof(T)}");

        // Ascending*/Descending* of RadixSortOperations.tt:30-125: (key type, descending)
        private static readonly Dictionary<Type, (int, bool)> SortOperations =
            new Dictionary<Type, (int, bool)>
        {
            { typeof(AscendingInt8), (I8, false) }, { typeof(DescendingInt8), (I8, true) },
            { typeof(AscendingInt16), (I16, false) }, { typeof(DescendingInt16), (I16, true) },
            { typeof(AscendingInt32), (I32, false) }, { typeof(DescendingInt32), (I32, true) },
            { typeof(AscendingInt64), (I64, false) }, { typeof(DescendingInt64), (I64, true) },
            { typeof(AscendingUInt8), (U8, false) }, { typeof(DescendingUInt8), (U8, true) },
            { typeof(AscendingUInt16), (U16, false) }, { typeof(DescendingUInt16), (U16, true) },
            { typeof(AscendingUInt32), (U32, false) }, { typeof(DescendingUInt32), (U32, true) },
            { typeof(AscendingUInt64), (U64, false) }, { typeof(DescendingUInt64), (U64, true) },
            { typeof(AscendingHalf), (F16, false) }, { typeof(DescendingHalf), (F16, true) },
            { typeof(AscendingFloat), (F32, false) }, { typeof(DescendingFloat), (F32, true) },
            { typeof(AscendingDouble), (F64, false) }, { typeof(DescendingDouble), (F64, true) },
        };

        /// <summary>Key type code and sort flags of a radix sort functor.</summary>
        public static (int KeyType, int Flags) SortOperation<T, TRadixSortOperation>()
            where T : unmanaged
            where TRadixSortOperation : struct, IRadixSortOperation<T>
        {
            if (!SortOperations.TryGetValue(typeof(TRadixSortOperation), out var entry))
                throw new NotSupportedException(
                    $"radix sort operation {typeof(TRadixSortOperation)}");
            if (entry.Item1 != ElementType<T>())
                throw new NotSupportedException("radix sort operation and key type differ");
            return (entry.Item1, entry.Item2 ? SortDescending : 0);
        }

        // Add/Max/Min x {Int32, Int64, UInt32, UInt64, Float, Double}
        // (ScanReduceOperations.tt:20-72)
        private static readonly Dictionary<Type, (int, int)> ScanReduceOperations =
            new Dictionary<Type, (int, int)>
        {
            { typeof(AddInt32), (I32, OpAdd) }, { typeof(MaxInt32), (I32, OpMax) },
            { typeof(MinInt32), (I32, OpMin) },
            { typeof(AddInt64), (I64, OpAdd) }, { typeof(MaxInt64), (I64, OpMax) },
            { typeof(MinInt64), (I64, OpMin) },
            { typeof(AddUInt32), (U32, OpAdd) }, { typeof(MaxUInt32), (U32, OpMax) },
            { typeof(MinUInt32), (U32, OpMin) },
            { typeof(AddUInt64), (U64, OpAdd) }, { typeof(MaxUInt64), (U64, OpMax) },
            { typeof(MinUInt64), (U64, OpMin) },
            { typeof(AddFloat), (F32, OpAdd) }, { typeof(MaxFloat), (F32, OpMax) },
            { typeof(MinFloat), (F32, OpMin) },
            { typeof(AddDouble), (F64, OpAdd) }, { typeof(MaxDouble), (F64, OpMax) },
            { typeof(MinDouble), (F64, OpMin) },
        };

        /// <summary>Element type code and operation code of a scan/reduce functor.</summary>
        public static (int ElementType, int Op) ScanReduceOperation<T, TOperation>()
            where T : unmanaged
            where TOperation : struct, IScanReduceOperation<T>
        {
            if (!ScanReduceOperations.TryGetValue(typeof(TOperation), out var entry))
                throw new NotSupportedException($"scan/reduce operation {typeof(TOperation)}");
            if (entry.Item1 != ElementType<T>())
                throw new NotSupportedException("scan/reduce operation and element type differ");
            return entry;
        }

        /// <summary>ScanKind to the native code.</summary>
        public static int Kind(ScanKind kind) =>
            kind == ScanKind.Inclusive ? ScanInclusive : ScanExclusive;

        // Identity sequencers: value = (T)index.  The integer ones truncate the
        // index (Sequencer.cs:36-45, Sequencers.tt:25-37), Half/Float/DoubleSequencer
        // convert it (Sequencer.cs:47-75).
        private static readonly Dictionary<Type, int> IndexSequencers = new Dictionary<Type, int>
        {
            { typeof(IndexSequencer), I32 },
            { typeof(Int8Sequencer), I8 }, { typeof(Int16Sequencer), I16 },
            { typeof(Int32Sequencer), I32 }, { typeof(Int64Sequencer), I64 },
            { typeof(UInt8Sequencer), U8 }, { typeof(UInt16Sequencer), U16 },
            { typeof(UInt32Sequencer), U32 }, { typeof(UInt64Sequencer), U64 },
            { typeof(HalfSequencer), F16 }, { typeof(FloatSequencer), F32 },
            { typeof(DoubleSequencer), F64 },
        };

        /// <summary>The element type an identity sequencer produces; any other
        /// sequencer (user code the reference would JIT-compile) is refused.</summary>
        public static int IndexSequencer<TValue, TSequencer>()
            where TValue : unmanaged
            where TSequencer : struct, ISequencer<TValue>
        {
            if (!IndexSequencers.TryGetValue(typeof(TSequencer), out int type))
                throw new NotSupportedException($"sequencer {typeof(TSequencer)}");
            if (type != ElementType<TValue>())
                throw new NotSupportedException("sequencer and value type differ");
            return type;
        }

        /// <summary>The value source of a key/value sort whose values an identity
        /// sequencer generates.</summary>
        public static int ValueSource<TValue, TSequencer>()
            where TValue : unmanaged
            where TSequencer : struct, ISequencer<TValue>
        {
            int type = IndexSequencer<TValue, TSequencer>();
            return type == F16 || type == F32 || type == F64
                ? ValuesFromIndexAsFloat
                : ValuesFromIndex;
        }

        // Comparison* of ComparisonOperations.tt:26-45: first.CompareTo(second).
        private static readonly Dictionary<Type, int> Comparisons =
            new Dictionary<Type, int>
        {
            { typeof(ComparisonInt8), I8 },
            { typeof(ComparisonInt16), I16 },
            { typeof(ComparisonInt32), I32 },
            { typeof(ComparisonInt64), I64 },
            { typeof(ComparisonUInt8), U8 },
            { typeof(ComparisonUInt16), U16 },
            { typeof(ComparisonUInt32), U32 },
            { typeof(ComparisonUInt64), U64 },
            { typeof(ComparisonHalf), F16 },
            { typeof(ComparisonFloat), F32 },
            { typeof(ComparisonDouble), F64 },
        };

        /// <summary>Element type code of a comparison functor of the reference.</summary>
        public static int ComparisonOperation<T, TComparisonOperation>()
            where T : unmanaged
            where TComparisonOperation : struct, IComparisonOperation<T>
        {
            if (!Comparisons.TryGetValue(typeof(TComparisonOperation), out int type))
                throw new NotSupportedException(
                    $"comparison operation {typeof(TComparisonOperation)}");
            if (type != ElementType<T>())
                throw new NotSupportedException("comparison operation and element type differ");
            return type;
        }

        /// <summary>Transformer code and factor of a transformer of this layer's closed
        /// set, or of the reference's IdentityTransformer (TransformExtensions.cs:42-55).
        /// </summary>
        public static (int Transformer, long Factor) Transformer<TSource, TTarget, TTransformer>(
            TTransformer transformer)
            where TSource : unmanaged
            where TTarget : unmanaged
            where TTransformer : struct, ITransformer<TSource, TTarget>
        {
            if (transformer is IHipTransformer known)
                return (known.Code, known.Factor);
            Type type = typeof(TTransformer);
            if (type.IsGenericType &&
                type.GetGenericTypeDefinition() == typeof(IdentityTransformer<>))
                return (TransformConvert, 0);
            throw new NotSupportedException($"transformer {type}");
        }

        /// <summary>Histogram locator code of a bin operation of this layer.</summary>
        public static int Locator<TLocator>() =>
            typeof(TLocator).IsGenericType &&
            typeof(TLocator).GetGenericTypeDefinition() == typeof(HipIdentityBinOperation<>)
            ? LocatorIdentity
            : typeof(TLocator).IsGenericType &&
              typeof(TLocator).GetGenericTypeDefinition() == typeof(HipModuloBinOperation<>)
            ? LocatorModulo
            : throw new NotSupportedException($"bin operation {typeof(TLocator)}");

        /// <summary>Bytes of a temp request as ArrayView&lt;int&gt; elements.</summary>
        public static long BytesToInts(long bytes) => (bytes + sizeof(int) - 1) / sizeof(int);
    }
}
