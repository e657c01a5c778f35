"""The C# P/Invoke layer (csharp/ILGPU.Algorithms.Hip) against the C header.

There is no .NET toolchain here, so the C# files cannot be compiled; what can
be checked mechanically is that every ``[DllImport]`` prototype names an
exported function, has the header's number of arguments and passes every
argument at the header's width, that no export is missing, and that the status
enum and the type codes agree with the header.
"""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ilgpu_hip_algorithms.h")
CSHARP = os.path.join(ROOT, "csharp", "ILGPU.Algorithms.Hip")


def strip_comments(text):
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(r"//[^\n]*", " ", text)


def header_prototypes():
    text = strip_comments(open(HEADER).read())
    protos = {}
    for m in re.finditer(r"\b(const\s+char\s*\*|int32_t|int64_t)\s*(ilgpu_hip_\w+)\s*\(([^;{]*?)\)\s*;",
                         text, flags=re.S):
        ret, name, params = m.group(1), m.group(2), " ".join(m.group(3).split())
        args = [] if params in ("", "void") else [p.strip() for p in params.split(",")]
        protos[name] = (" ".join(ret.split()), args)
    return protos


def c_width(decl):
    """'ptr', 'i32', 'i64' of a C parameter declaration or return type."""
    if "*" in decl or decl.startswith("ilgpu_hip_stream_t"):
        return "ptr"
    if decl.startswith("int32_t"):
        return "i32"
    if decl.startswith("int64_t"):
        return "i64"
    raise AssertionError(f"unexpected C type in {decl!r}")


def cs_width(decl):
    """The same for a C# parameter declaration or return type."""
    decl = decl.strip()
    type_part = decl.rsplit(" ", 1)[0] if " " in decl else decl
    if "*" in type_part or type_part.startswith("out ") or type_part in ("IntPtr", "string"):
        return "ptr"
    if type_part == "int":
        return "i32"
    if type_part == "long":
        return "i64"
    raise AssertionError(f"unexpected C# type in {decl!r}")


def csharp_prototypes():
    text = strip_comments(open(os.path.join(CSHARP, "HipAlgorithmsNativeMethods.cs")).read())
    protos = {}
    pattern = r"\[DllImport\(LibName[^\]]*\)\]\s*internal\s+static\s+extern\s+(\w+)\s+(\w+)\s*\(([^)]*)\)\s*;"
    for m in re.finditer(pattern, text, flags=re.S):
        ret, name, params = m.group(1), m.group(2), " ".join(m.group(3).split())
        args = [] if not params else [p.strip() for p in params.split(",")]
        assert name not in protos, f"{name} imported twice"
        protos[name] = (ret, args)
    return protos


def test_every_export_is_imported_once_and_nothing_else():
    c, cs = header_prototypes(), csharp_prototypes()
    from ilgpu_amd import capi
    assert sorted(c) == sorted(capi.EXPORTS)      # the parser saw every declaration
    assert sorted(cs) == sorted(c)
    text = open(os.path.join(CSHARP, "HipAlgorithmsNativeMethods.cs")).read()
    assert 'LibName = "libilgpu_hip_algorithms.so"' in text
    assert text.count("[DllImport(") == len(c)


def test_every_prototype_has_the_headers_arity_and_widths():
    c, cs = header_prototypes(), csharp_prototypes()
    for name, (c_ret, c_args) in c.items():
        cs_ret, cs_args = cs[name]
        assert len(cs_args) == len(c_args), (name, cs_args, c_args)
        assert cs_width(cs_ret) == c_width(c_ret), (name, "return")
        for i, (a, b) in enumerate(zip(cs_args, c_args)):
            assert cs_width(a) == c_width(b), (name, i, a, b)


def test_single_value_results_are_out_parameters_of_the_right_width():
    # int64_t* results written by the call on the host are `out long`; a double* is `out double`
    cs = csharp_prototypes()
    for name in ("ilgpu_hip_radix_sort_temp_bytes", "ilgpu_hip_radix_sort_temp_bytes_strided",
                 "ilgpu_hip_scan_temp_bytes", "ilgpu_hip_reduce_temp_bytes",
                 "ilgpu_hip_unique_temp_bytes"):
        assert cs[name][1][-1].startswith("out long "), name
    assert cs["ilgpu_hip_profile_query"][1][1].startswith("out long ")
    assert cs["ilgpu_hip_profile_query"][1][2].startswith("out double ")
    # device pointers are never marshalled as out/ref
    for name in ("ilgpu_hip_unique", "ilgpu_hip_selftest_lds_atomic_order", "ilgpu_hip_histogram"):
        assert not any(a.startswith(("out ", "ref ")) for a in cs[name][1]), name


def header_enum(prefix):
    text = strip_comments(open(HEADER).read())
    return {m.group(1): int(m.group(2))
            for m in re.finditer(r"\b(" + prefix + r"\w+)\s*=\s*(\d+)", text)}


def test_status_enum_and_type_codes_match_the_header():
    status = header_enum("ILGPU_HIP_ERROR_")
    status["ILGPU_HIP_SUCCESS"] = 0
    text = open(os.path.join(CSHARP, "HipAlgorithmsException.cs")).read()
    cs_status = {m.group(1): int(m.group(2))
                 for m in re.finditer(r"^\s+(\w+) = (\d+),", text, flags=re.M)}
    expect = {"Success": "ILGPU_HIP_SUCCESS", "NullView": "ILGPU_HIP_ERROR_NULL_VIEW",
              "OutOfRange": "ILGPU_HIP_ERROR_OUT_OF_RANGE",
              "NotSupported": "ILGPU_HIP_ERROR_NOT_SUPPORTED",
              "UnalignedTemp": "ILGPU_HIP_ERROR_UNALIGNED_TEMP", "Runtime": "ILGPU_HIP_ERROR_RUNTIME",
              "StaticLimit": "ILGPU_HIP_ERROR_STATIC_LIMIT"}
    assert set(cs_status) == set(expect) and len(status) == len(expect)
    for cs_name, c_name in expect.items():
        assert cs_status[cs_name] == status[c_name], cs_name

    type_map = open(os.path.join(CSHARP, "HipTypeMap.cs")).read()
    consts = {m.group(1): int(m.group(2)) for m in re.finditer(r"\b(\w+) = (\d+)\b", type_map)}
    types = header_enum("ILGPU_HIP_[IUF](?:8|16|32|64)")
    for c_name, value in types.items():
        assert consts[c_name[len("ILGPU_HIP_"):]] == value, c_name
    others = {"OpAdd": "ILGPU_HIP_OP_ADD", "OpMax": "ILGPU_HIP_OP_MAX", "OpMin": "ILGPU_HIP_OP_MIN",
              "ScanInclusive": "ILGPU_HIP_SCAN_INCLUSIVE", "ScanExclusive": "ILGPU_HIP_SCAN_EXCLUSIVE",
              "SortDescending": "ILGPU_HIP_SORT_DESCENDING",
              "SortFloatTotalOrder": "ILGPU_HIP_SORT_FLOAT_TOTAL_ORDER",
              "ValuesFromView": "ILGPU_HIP_VALUES_FROM_VIEW",
              "ValuesFromIndex": "ILGPU_HIP_VALUES_FROM_INDEX",
              "LocatorIdentity": "ILGPU_HIP_LOCATOR_IDENTITY",
              "LocatorModulo": "ILGPU_HIP_LOCATOR_MODULO"}
    all_header = header_enum("ILGPU_HIP_")
    for cs_name, c_name in others.items():
        assert consts[cs_name] == all_header[c_name], cs_name


def test_functor_tables_cover_every_built_in_functor():
    # RadixSortOperations.tt: Ascending/Descending x 11 numeric types;
    # ScanReduceOperations.tt: Add/Max/Min x 6 atomic numeric types
    text = open(os.path.join(CSHARP, "HipTypeMap.cs")).read()
    names = ["Int8", "Int16", "Int32", "Int64", "UInt8", "UInt16", "UInt32", "UInt64", "Half",
             "Float", "Double"]
    for n in names:
        assert f"typeof(Ascending{n})" in text and f"typeof(Descending{n})" in text, n
    for n in ["Int32", "Int64", "UInt32", "UInt64", "Float", "Double"]:
        for op in ("Add", "Max", "Min"):
            assert f"typeof({op}{n})" in text, (op, n)


def test_public_surface_names_the_references_methods():
    def has(file, *names):
        text = open(os.path.join(CSHARP, file)).read()
        for n in names:
            assert re.search(r"public static [^;{]*\b" + n + r"\s*<", text) or \
                re.search(r"public static [^;{]*\b" + n + r"\s*\(", text), (file, n)
    has("HipRadixSortExtensions.cs", "CreateRadixSort", "CreateRadixSortPairs",
        "ComputeRadixSortTempStorageSize", "ComputeRadixSortPairsTempStorageSize",
        "CreateRadixSortProvider")
    has("HipScanExtensions.cs", "CreateScan", "ComputeScanTempStorageSize", "CreateScanProvider")
    has("HipReductionExtensions.cs", "CreateReduction", "Reduce", "ReduceAsync")
    has("HipHistogramExtensions.cs", "CreateHistogram", "CreateHistogramUnchecked", "Histogram",
        "HistogramUnchecked")


def test_every_import_is_used_by_the_layers_public_surface():
    # A DllImport nobody calls is an entry point C# users cannot reach.  The one
    # exception is deliberate: ilgpu_hip_sort_set_parameter is a process-wide
    # test hook of the library and stays out of the public surface.
    hidden = {"ilgpu_hip_sort_set_parameter"}
    others = ""
    for name in sorted(os.listdir(CSHARP)):
        if name.endswith(".cs") and name != "HipAlgorithmsNativeMethods.cs":
            others += strip_comments(open(os.path.join(CSHARP, name)).read())
    for name in csharp_prototypes():
        used = re.search(r"\b" + name + r"\s*\(", others) is not None
        assert used != (name in hidden), name


def test_reference_surface_of_the_neighbouring_primitives_is_there():
    # Unique, Initialize, Sequence, Reorder and Transform: every public method of
    # the reference's extension classes has a counterpart of the same name.
    expected = {
        "HipUniqueExtensions.cs": ["ComputeUniqueTempStorageSize", "CreateUnique", "Unique"],
        "HipInitializeExtensions.cs": ["CreateInitializer", "Initialize"],
        "HipSequenceExtensions.cs": ["CreateSequencer", "CreateBatchedSequencer",
                                     "CreateRepeatedSequencer", "CreateRepeatedBatchedSequencer",
                                     "Sequence", "RepeatedSequence", "BatchedSequence",
                                     "RepeatedBatchedSequence"],
        "HipReorderExtensions.cs": ["CreateReorderTransformer", "Reorder", "ReorderTransform"],
        "HipTransformExtensions.cs": ["CreateTransformer", "Transform"],
    }
    for file_name, methods in expected.items():
        text = strip_comments(open(os.path.join(CSHARP, file_name)).read())
        for method in methods:
            assert re.search(r"public\s+static\s+[^;{(]*\b" + method + r"\s*<", text, flags=re.S), \
                (file_name, method)
    type_map = open(os.path.join(CSHARP, "HipTypeMap.cs")).read()
    for functor in ["ComparisonInt8", "ComparisonUInt64", "ComparisonHalf", "ComparisonDouble",
                    "Int8Sequencer", "UInt16Sequencer", "HalfSequencer", "FloatSequencer",
                    "DoubleSequencer", "IdentityTransformer"]:
        assert functor in type_map, functor
