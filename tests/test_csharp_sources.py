"""The managed half of the backend (csharp/TensorSharp.HIP/*.cs) cannot be compiled here (no .NET in the image); what can
be checked on the text is checked: every function the C header declares has exactly one [DllImport] with the same
number of parameters, every DllImport names a declared function, every op name of the decode path has exactly one
handler registered for HipStorage with the CPU backend's parameter count, and the marshalled structs have the header's
field order."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CS = os.path.join(ROOT, "csharp", "TensorSharp.HIP")


def _split_args(s):
    out, depth, cur = [], 0, ""
    for ch in s:
        if ch in "([<":
            depth += 1
        elif ch in ")]>":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur)
            cur = ""
        else:
            cur += ch
    if cur.strip() and cur.strip() != "void":
        out.append(cur)
    return out


def _header_functions():
    text = open(os.path.join(ROOT, "include", "tship.h")).read()
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    fns = {}
    for m in re.finditer(r"TSHIP_API\s+[\w\s\*]+?\b(TSHip_\w+)\s*\((.*?)\)\s*;", text, flags=re.S):
        fns[m.group(1)] = len(_split_args(m.group(2)))
    return fns


def _dll_imports():
    text = open(os.path.join(CS, "HipNative.cs")).read()
    text = re.sub(r"//.*", "", text)
    found = []
    for m in re.finditer(r"\[DllImport\([^\]]*\)\]\s*(?:private|internal|public)\s+static\s+extern\s+(?:unsafe\s+)?\w+\s+(TSHip_\w+)\s*\((.*?)\)\s*;", text, flags=re.S):
        found.append((m.group(1), len(_split_args(m.group(2)))))
    return found


def test_every_export_has_exactly_one_dllimport_with_the_same_arity():
    header = _header_functions()
    imports = _dll_imports()
    assert len(header) >= 60
    names = [n for n, _ in imports]
    assert sorted(set(names)) == sorted(names), "a function is imported twice"
    assert sorted(names) == sorted(header), (sorted(set(header) - set(names)), sorted(set(names) - set(header)))
    for n, argc in imports:
        assert argc == header[n], (n, argc, header[n])


# the op names the decode path issues, with the CPU handlers' parameter counts (TensorSharp/Ops.cs, Cpu/CpuBasicOps.cs,
# CpuIndexingOps.cs, CpuFillCopyOps.cs)
HOT_PATH_OPS = {
    "fill": 2, "addmm": 6, "addmmbatch": 6, "indexselect": 4, "indexselectgrad": 3, "rope": 4, "rmsnorm": 5, "layernorm": 5,
    "softmax": 2, "argmax": 3, "topK": 4, "addt": 3, "subt": 3, "mult": 3, "divt": 3, "addv": 3, "subv": 3, "mulv": 3, "divv": 3,
    "relu": 2, "SiLU": 2, "LeakyReLU": 2, "exp": 2, "log": 2, "neg": 2, "sigmoid": 2, "tanh": 2, "sqrt": 2, "abs": 2,
    "float2half": 2, "half2float": 2, "buildtrimask": 3, "buildselftrimask": 5, "iscorrupted": 1, "gather": 4, "scatter_fill": 4,
}


def test_every_hot_path_op_has_one_handler_registered_for_hip_storage():
    text = open(os.path.join(CS, "HipBasicOps.cs")).read()
    text = re.sub(r"//.*", "", text)
    assert "[OpsClass]" in text
    reg = re.findall(r'\[RegisterOpStorageType\("(\w+)",\s*typeof\(HipStorage\)\)\]\s*public\s+(?:static\s+)?(?:unsafe\s+)?[\w\[\]]+\s+\w+\s*\((.*?)\)', text, flags=re.S)
    names = [n for n, _ in reg]
    assert sorted(names) == sorted(set(names)), "an op is registered twice"
    assert sorted(names) == sorted(HOT_PATH_OPS), (sorted(set(HOT_PATH_OPS) - set(names)), sorted(set(names) - set(HOT_PATH_OPS)))
    for n, args in reg:
        assert len(_split_args(args)) == HOT_PATH_OPS[n], n
    # "copy" is registered by argument count with per-parameter storage types: device/device, host/device, device/host
    copies = re.findall(r'\[RegisterOpArgCount\("copy"\)\]\s*public\s+void\s+\w+\s*\(\s*\[OpArgStorageType\(typeof\((\w+)\)\)\]\s*Tensor\s+result,\s*\[OpArgStorageType\(typeof\((\w+)\)\)\]\s*Tensor\s+src\)', text)
    assert sorted(copies) == sorted([("HipStorage", "HipStorage"), ("HipStorage", "CpuStorage"), ("CpuStorage", "HipStorage")])


def test_marshalled_structs_follow_the_header():
    h = re.sub(r"/\*.*?\*/", " ", open(os.path.join(ROOT, "include", "tship.h")).read(), flags=re.S)
    cs = re.sub(r"//.*", "", open(os.path.join(CS, "HipNative.cs")).read())
    cfg_h = re.search(r"typedef struct TSHipGptConfig \{(.*?)\} TSHipGptConfig;", h, flags=re.S).group(1)
    fields_h = [f.strip().lstrip("*") for decl in cfg_h.split(";") if decl.strip() for f in decl.strip().split(None, 1)[1].split(",")]
    types_h = []
    for decl in cfg_h.split(";"):
        if decl.strip():
            t, names = decl.strip().split(None, 1)
            types_h += [t] * len(names.split(","))
    cfg_cs = re.search(r"public struct TSHipGptConfig\s*\{(.*?)\}", cs, flags=re.S).group(1)
    types_cs = []
    for decl in cfg_cs.split(";"):
        d = decl.strip()
        if d.startswith("public"):
            _, t, names = d.split(None, 2)
            types_cs += [t] * len(names.split(","))
    assert len(fields_h) == len(types_cs) == 19
    assert [{"int32_t": "int", "float": "float"}[t] for t in types_h] == types_cs
    ten = re.search(r"internal unsafe struct TSHipTensor\s*\{(.*?)public static", cs, flags=re.S).group(1)
    order = re.findall(r"public\s+(?:fixed\s+)?(\w+)\s+(\w+)", ten)
    assert order == [("IntPtr", "Data"), ("int", "DType"), ("int", "NDim"), ("long", "Sizes"), ("long", "Strides")]
    assert "Sizes[6]" in ten and "Strides[6]" in ten and "#define TSHIP_MAX_DIMS 6" in h


def test_backend_classes_implement_the_reference_interfaces():
    storage = open(os.path.join(CS, "HipStorage.cs")).read()
    for member in ["GetElementsAsInt", "SetElementsAsInt", "LocationDescription", "GetElementAsFloat", "GetElementsAsFloat", "SetElementAsFloat",
                   "SetElementsAsFloat", "SetElementsAsHalf", "CopyToStorage", "CopyFromStorage", "Destroy"]:      # TensorSharp/Storage.cs:32-47, RefCounted
        assert re.search(r"override\s+(?:unsafe\s+)?[\w\[\]]+\s+%s\s*\(" % member, storage), member
    alloc = open(os.path.join(CS, "HipAllocator.cs")).read()
    for member in ["BlasEnum BlasEnum", "int DeviceId", "Storage Allocate(DType elementType, long elementCount)", "float GetAllocatedMemoryRatio()"]:   # IAllocator.cs:13-20
        assert member in alloc, member
    ctx = open(os.path.join(CS, "HipContext.cs")).read()
    assert "OpRegistry.RegisterAssembly(Assembly.GetExecutingAssembly())" in ctx


def _strip_cs(text):
    """C# source without comments, string and character literals (enough for a bracket check)."""
    out, i, n = [], 0, len(text)
    while i < n:
        ch = text[i]
        if text.startswith("//", i):
            i = text.find("\n", i)
            i = n if i < 0 else i
        elif text.startswith("/*", i):
            i = text.find("*/", i) + 2
        elif ch == '"':
            verbatim = i > 0 and text[i - 1] == "@"
            i += 1
            while i < n:
                if verbatim and text.startswith('""', i):
                    i += 2
                elif not verbatim and text[i] == "\\":
                    i += 2
                elif text[i] == '"':
                    break
                else:
                    i += 1
            i += 1
        elif ch == "'":
            i = text.find("'", i + 2 if text[i + 1] == "\\" else i + 1) + 1
        else:
            out.append(ch)
            i += 1
    return "".join(out)


def test_sources_are_bracket_balanced_and_call_only_declared_natives():
    """No compiler is at hand, so at least: every bracket closes in every file, every `HipNative.X(` call names a declared
    import, and every statement-level call of a status-returning import goes through Check."""
    import glob
    declared = set(re.findall(r"static extern (?:unsafe )?\w+\*? (TSHip_\w+)\(", open(os.path.join(CS, "HipNative.cs")).read()))
    assert len(declared) >= 60
    for path in sorted(glob.glob(os.path.join(CS, "*.cs"))):
        code = _strip_cs(open(path).read())
        stack = []
        pairs = {")": "(", "]": "[", "}": "{"}
        for ch in code:
            if ch in "([{":
                stack.append(ch)
            elif ch in pairs:
                assert stack and stack.pop() == pairs[ch], path
        assert not stack, path
        for name in re.findall(r"HipNative\.(TSHip_\w+)\(", code):
            assert name in declared, (path, name)
