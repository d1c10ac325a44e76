"""The C-ABI library loads without a GPU and exports every symbol the headers under include/ declare."""
import ctypes
import os
import re
import subprocess

from libnd4j_amd import native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_c_names():
    text = open(os.path.join(ROOT, "include", "nd4j_native_c.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = text.replace("\\\n", " ")
    names = set(re.findall(r"\b(nd4j_(?:amd_)?[A-Za-z0-9]+)\s*\(", text))
    for macro_name in ("ND4J_C_EXEC", "ND4J_C_SCALAR", "ND4J_C_REDUCE3", "ND4J_C_SPECIAL"):
        macro = re.search(r"#define %s\(SUFFIX, T(?:, [RS])?\)(.*?)\n\s*\n" % macro_name, text, flags=re.S).group(1)
        for templ in re.findall(r"\b(nd4j_[A-Za-z0-9#]+)\s*\(", macro):
            for suffix in ("Float", "Half", "Double"):
                names.add(templ.replace("##SUFFIX##", suffix).replace("##SUFFIX", suffix))
    return {n for n in names if "#" not in n}


def test_library_loads_and_exports_every_declared_symbol():
    lib = native.load_library()
    declared = _declared_c_names()
    assert len(declared) > 90
    for name in sorted(declared):
        assert hasattr(lib, name), "missing export " + name
    assert set(native.exported_symbol_names()) <= declared | {"nd4j_lastError"}


def test_cpp_class_members_are_exported():
    out = subprocess.check_output(["nm", "-DC", "--defined-only", native.LIBRARY_PATH]).decode()
    for member in ("execTransformFloat", "execTransformHalf", "execPairwiseTransformFloat", "execBroadcastFloat",
                   "execReduceFloat", "execReduceScalarFloat", "execIndexReduceFloat", "execIndexReduceScalarFloat",
                   "execSummaryStatsFloat", "execSummaryStatsScalarFloat", "execRandomFloat", "execRandomHalf",
                   "execScalarFloat", "execScalarHalf", "execScalarDouble", "execReduce3Float", "execReduce3ScalarFloat",
                   "execReduce3AllFloat", "execReduce3Half", "execReduce3Double", "flattenFloat", "concatFloat", "concatHalf",
                   "pullRowsFloat", "pullRowsDouble", "tearFloat", "shuffleFloat", "shuffleHalf", "convertTypes",
                   "initRandom", "refreshBuffer", "reSeedBuffer", "destroyRandom", "tadOnlyShapeInfo", "mallocDevice",
                   "createStream", "memcpyAsync", "streamSynchronize"):
        assert "NativeOps::%s(" % member in out, member
    # the mangled name a JavaCPP binding generated from the reference header would look up
    raw = subprocess.check_output(["nm", "-D", "--defined-only", native.LIBRARY_PATH]).decode()
    assert "_ZN9NativeOps18execTransformFloatEPPviPfxS2_xS2_x" in raw
    assert "_ZN9NativeOps17execTransformHalfEPPviP7float16PxS3_S4_S3_" in raw


def test_last_error_is_empty_after_a_host_only_call():
    ops = native.NativeOps()
    ops.setGridLimit(128)
    assert ops._lib.nd4j_lastError() == b""
    assert ops.ompGetMaxThreads() >= 32


def test_missing_library_fails_loudly(tmp_path):
    import pytest
    with pytest.raises(ImportError):
        native.load_library(str(tmp_path / "nope.so"))


def test_every_member_of_the_reference_class_is_exported():
    """The reference's CPU back end, compiled where it lies for the checker (oracle/_ref/NativeOps.o), defines every
    member of class NativeOps; each of those mangled names must be a defined export of this library, so that a
    binding generated from the reference's header links against it."""
    import pytest
    ref_obj = os.path.join(ROOT, "oracle", "_ref", "NativeOps.o")
    if not os.path.exists(ref_obj):
        pytest.skip("oracle/_ref/NativeOps.o not built (needs the reference tree)")

    def members(path, dynamic):
        out = subprocess.check_output(["nm", "--defined-only"] + (["-D"] if dynamic else []) + [path]).decode()
        return {line.split()[-1] for line in out.splitlines() if " T _ZN9NativeOps" in line}

    want, have = members(ref_obj, False), members(native.LIBRARY_PATH, True)
    assert len(want) > 200
    assert not (want - have), sorted(want - have)[:5]
