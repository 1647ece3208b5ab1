"""The OCaml side of the plugin (ocaml/sarek-hip/*.ml) cannot be compiled here: there is no OCaml toolchain.
What can be checked without one is checked here, mechanically: every ctypes stub names a symbol of
include/sarek_hip.h with that symbol's signature, the struct declarations list the header's members in the
header's order, the ABI version the veneer expects is the header's, the dune file lists the modules that exist,
and every file is lexically sound OCaml (comments, strings and brackets closed)."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
OCAML = os.path.join(ROOT, "ocaml", "sarek-hip")
HEADER = os.path.join(ROOT, "include", "sarek_hip.h")

HANDLES = {"sarek_hip_stream": "void *", "sarek_hip_event": "void *", "sarek_hip_kernel": "void *",
           "sarek_hip_vector": "void *"}


def header_text():
    return re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)


def normalise_c(param):
    """'const float *a' -> 'float *', 'const int block[3]' -> 'int *', 'sarek_hip_stream s' -> 'void *'."""
    p = " ".join(param.split())
    array = bool(re.search(r"\[\d*\]\s*$", p))
    p = re.sub(r"\[\d*\]\s*$", "", p)
    p = re.sub(r"\bconst\b", "", p)
    stars = p.count("*")
    words = p.replace("*", " ").split()
    if len(words) > 1 and words[-1] not in ("int", "char", "float", "double", "void", "unsigned", "size_t") \
            and not words[-1].endswith("_t") and not words[-1].startswith("sarek_hip_"):
        words = words[:-1]                       # the parameter's name
    base = " ".join(words)
    if base in HANDLES:
        base, stars = "void", stars + 1
    return (base + " " + "*" * (stars + (1 if array else 0))).strip()


def header_prototypes():
    protos = {}
    for m in re.finditer(r"^([\w \*]+?)\b(sarek_hip_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", header_text(), flags=re.M | re.S):
        ret = normalise_c(m.group(1) + " x") if m.group(1).strip() != "int" else "int"
        args = [a for a in (s.strip() for s in m.group(3).split(",")) if a]
        protos[m.group(2)] = (ret, [] if args == ["void"] else [normalise_c(a) for a in args])
    return protos


OCAML_SCALARS = {"int": "int", "uint": "unsigned", "uchar": "unsigned char", "size_t": "size_t", "int64_t": "int64_t",
                 "int32_t": "int32_t", "uint64_t": "uint64_t", "uint32_t": "uint32_t", "uint16_t": "uint16_t", "float": "float",
                 "double": "double", "char": "char", "void": "void", "string": "char *",
                 "arg": "sarek_hip_arg", "launch": "sarek_hip_launch", "device_info": "sarek_hip_device_info"}


def c_of_ocaml(t):
    """'ptr (ptr void)' -> 'void **', 'string' -> 'char *', 'ptr arg' -> 'sarek_hip_arg *'."""
    t = t.strip()
    while t.startswith("(") and t.endswith(")"):
        t = t[1:-1].strip()
    if t.startswith("ptr "):
        inner = c_of_ocaml(t[4:])
        return inner + ("*" if inner.endswith("*") else " *")
    return OCAML_SCALARS[t]


def ocaml_stubs():
    text = open(os.path.join(OCAML, "Hip_bindings.ml")).read()
    text = re.sub(r"\(\*.*?\*\)", "", text, flags=re.S)
    stubs = {}
    for m in re.finditer(r'bind\s+"(sarek_hip_\w+)"\s*\((.*?returning\s+\w+)\)', text, flags=re.S):
        parts = [p.strip() for p in " ".join(m.group(2).split()).split("@->")]
        ret = parts[-1].replace("returning", "").strip()
        args = parts[:-1]
        stubs[m.group(1)] = (c_of_ocaml(ret), [] if args == ["void"] else [c_of_ocaml(a) for a in args])
    return stubs


def squeeze(t):
    return t.replace(" ", "")


def test_every_stub_binds_a_header_symbol_with_its_signature():
    protos, stubs = header_prototypes(), ocaml_stubs()
    assert len(stubs) >= 75
    for name, (ret, args) in stubs.items():
        assert name in protos, f"{name} is not declared in include/sarek_hip.h"
        pret, pargs = protos[name]
        assert squeeze(ret) == squeeze(pret), (name, ret, pret)
        assert [squeeze(a) for a in args] == [squeeze(a) for a in pargs], (name, args, pargs)


def test_the_backend_level_entry_points_are_all_bound():
    """Everything Framework_sig.BACKEND needs from the library, plus the library kernels and the kernel list."""
    stubs = ocaml_stubs()
    need = ["init", "is_available", "device_count", "device_get_info", "device_info_size", "device_set_current",
            "device_synchronize", "mem_alloc", "mem_free", "memcpy_htod", "memcpy_dtoh", "memcpy_dtod",
            "mem_alloc_zero_copy", "host_alloc", "host_free", "stream_create", "stream_destroy",
            "stream_synchronize", "event_create", "event_destroy", "event_record", "event_synchronize",
            "event_elapsed_ms", "kernel_compile", "kernel_compile_cached", "kernel_clear_cache", "kernel_launch",
            "profiler_start", "profiler_stop", "generate_source", "run_source", "run_sources",
            "intrinsic_register", "intrinsic_find", "intrinsic_list", "library_kernel_source",
            "library_kernel_list", "abi_version", "last_error", "status_name"]
    assert [n for n in need if "sarek_hip_" + n not in stubs] == []


def header_struct(name):
    body = re.search(r"typedef struct[^{]*\{([^}]*)\}\s*" + name + r"\s*;", header_text(), flags=re.S).group(1)
    fields = []
    for decl in body.split(";"):
        decl = " ".join(decl.split())
        if not decl:
            continue
        m = re.match(r"(.*?)(\w+(?:\[\d+\])?(?:\s*,\s*\w+(?:\[\d+\])?)*)$", decl)
        ctype = " ".join(m.group(1).replace("const", "").split())
        for n in m.group(2).split(","):
            n = n.strip()
            a = re.fullmatch(r"(\w+)\[(\d+)\]", n)
            fields.append((a.group(1), ctype, int(a.group(2))) if a else (n, ctype, None))
    return fields


def ocaml_struct(var):
    text = open(os.path.join(OCAML, "Hip_bindings.ml")).read()
    out = []
    for m in re.finditer(r'field ' + var + r' "(\w+)" (\(array (\d+) (\w+)\)|\(ptr \w+\)|\w+)', text):
        if m.group(3):
            out.append((m.group(1), OCAML_SCALARS[m.group(4)], int(m.group(3))))
        else:
            out.append((m.group(1), c_of_ocaml(m.group(2)), None))
    assert re.search(r"let \(\) = seal " + var + r"\b", text)
    return out


@pytest.mark.parametrize("var,cname", [("device_info", "sarek_hip_device_info"), ("arg", "sarek_hip_arg"),
                                       ("launch", "sarek_hip_launch")])
def test_struct_declarations_follow_the_header(var, cname):
    want = [(n, squeeze(t), k) for n, t, k in header_struct(cname)]
    got = [(n, squeeze(t), k) for n, t, k in ocaml_struct(var)]
    assert got == want


def test_expected_abi_version_is_the_headers():
    import __graft_entry__ as entry
    api = open(os.path.join(OCAML, "Hip_api.ml")).read()
    assert int(re.search(r"let expected_abi_version = (\d+)", api).group(1)) == entry.header_abi_version()
    assert "device_info_size" in api and "sizeof Hip_bindings.device_info" in api


def test_dune_lists_the_modules_that_exist():
    dune = open(os.path.join(OCAML, "dune")).read()
    listed = re.search(r"\(modules([^)]*)\)", dune).group(1).split()
    files = sorted(f[:-3] for f in os.listdir(OCAML) if f.endswith(".ml"))
    assert sorted(listed) == files
    assert "(name sarek_hip)" in dune and "(public_name sarek-hip.plugin)" in dune


def lex_ocaml(text):
    """Walk OCaml source: nested comments (strings inside comments count, as the compiler has it), strings,
    character literals, bracket balance.  Returns the code with comments and literals blanked."""
    out, i, n, depth, stack = [], 0, len(text), 0, []
    pairs = {")": "(", "]": "[", "}": "{"}
    while i < n:
        c = text[i]
        two = text[i:i + 2]
        if two == "(*" and text[i:i + 3] != "(*)":
            depth += 1
            i += 2
            continue
        if depth and two == "*)":
            depth -= 1
            i += 2
            continue
        if c == '"':
            j = i + 1
            while j < n and text[j] != '"':
                j += 2 if text[j] == "\\" else 1
            assert j < n, f"unterminated string starting at offset {i}: {text[i:i + 40]!r}"
            i = j + 1
            if not depth:
                out.append('""')
            continue
        if c == "'" :
            m = re.match(r"'(\\.|\\[0-9]{3}|[^\\'])'", text[i:])
            if m:
                i += m.end()
                if not depth:
                    out.append("' '")
                continue
        if not depth:
            if c in "([{":
                stack.append(c)
            elif c in ")]}":
                assert stack and stack[-1] == pairs[c], f"unbalanced {c!r} at offset {i}: {text[max(0, i - 40):i + 1]!r}"
                stack.pop()
            out.append(c)
        i += 1
    assert depth == 0, "comment not closed"
    assert stack == [], f"brackets left open: {stack}"
    return "".join(out)


def ocaml_files():
    found = []
    for d, _, files in os.walk(os.path.join(ROOT, "ocaml")):
        found += [os.path.join(d, f) for f in files if f.endswith(".ml")]
    return sorted(found)


def test_every_ocaml_file_is_lexically_sound():
    files = ocaml_files()
    assert len(files) >= 8
    for path in files:
        code = lex_ocaml(open(path).read())
        # keyword pairs that must balance in a file that compiles
        words = re.findall(r"\b(struct|sig|begin|object|end)\b", code)
        assert words.count("end") == len(words) - words.count("end"), path


def test_plugin_implements_every_member_of_the_backend_signature():
    """Names Framework_sig.BACKEND asks for (spoc/framework/Framework_sig.ml:146-350), looked for in the two
    plugin modules (written out here: the reference tree is not available where the tests run)."""
    base = lex_ocaml(open(os.path.join(OCAML, "Hip_plugin_base.ml")).read())
    plugin = lex_ocaml(open(os.path.join(OCAML, "Hip_plugin.ml")).read())
    members = {
        "": ["name", "version", "is_available", "enable_profiling", "disable_profiling"],
        "Device": ["init", "count", "get", "id", "name", "capabilities", "set_current", "synchronize"],
        "Stream": ["create", "destroy", "synchronize", "default"],
        "Memory": ["alloc", "alloc_custom", "alloc_zero_copy", "free", "host_to_device", "device_to_host",
                   "host_ptr_to_device", "device_to_host_ptr", "device_to_device", "size", "device_ptr", "is_zero_copy"],
        "Event": ["create", "destroy", "record", "synchronize", "elapsed"],
        "Kernel": ["compile", "compile_cached", "clear_cache", "create_args", "set_arg_buffer", "set_arg_int32",
                   "set_arg_int64", "set_arg_float32", "set_arg_float64", "set_arg_ptr", "launch"],
    }
    for module, names in members.items():
        if module:
            body = re.search(r"module " + module + r" = struct(.*?)\n  end", base, flags=re.S).group(1)
        else:
            body = base
        for name in names:
            assert re.search(r"\blet " + name + r"\b", body), (module, name)
    for name in ["execution_model", "generate_source", "execute_direct", "supported_source_langs", "run_source",
                 "wrap_kargs", "unwrap_kargs"]:
        assert re.search(r"\blet " + name + r"\b", plugin), name
    assert "module Intrinsics = Hip_intrinsics" in plugin
    for name in ["register", "find", "list_all"]:
        assert re.search(r"\blet " + name + r"\b", plugin), name
    caps = ["max_threads_per_block", "max_block_dims", "max_grid_dims", "shared_mem_per_block", "total_global_mem",
            "compute_capability", "supports_fp64", "supports_atomics", "warp_size", "max_registers_per_block",
            "clock_rate_khz", "multiprocessor_count", "is_cpu"]
    cap_body = re.search(r"let capabilities.*?\n      \}", base, flags=re.S).group(0)
    assert [c for c in caps if not re.search(r"\b" + c + r" =", cap_body)] == []


def test_serialiser_prints_only_forms_the_native_reader_knows():
    """Every form head and atom Sarek_ir_hip.ml can print ("(read", "(lelemx", "bitxor", "downto", ...) is a
    literal of the reader (spoc_amd/csrc/host/ir_text.cpp), so the two cannot drift apart unnoticed."""
    ml = open(os.path.join(OCAML, "Sarek_ir_hip.ml")).read()
    reader = open(os.path.join(ROOT, "spoc_amd", "csrc", "host", "ir_text.cpp")).read()
    heads = sorted(set(re.findall(r'"\((\w+)', ml)))
    atoms = sorted(set(re.findall(r'-> "([a-z_0-9]+)"', ml)))
    assert len(heads) >= 45 and len(atoms) >= 30
    assert [w for w in heads + atoms if f'"{w}"' not in reader] == []
    # one printer per IR type, one case per constructor of spoc/ir/Sarek_ir_types.ml
    constructors = ["TInt32", "TInt64", "TFloat32", "TFloat64", "TBool", "TUnit", "TRecord", "TVariant", "TArray",
                    "TVec", "CInt32", "CInt64", "CFloat32", "CFloat64", "CBool", "CUnit", "EConst", "EVar", "EBinop",
                    "EUnop", "EArrayRead", "EArrayReadExpr", "ERecordField", "EIntrinsic", "ECast", "ETuple", "EApp",
                    "ERecord", "EVariant", "EArrayLen", "EArrayCreate", "EIf", "EMatch", "LVar", "LArrayElem",
                    "LArrayElemExpr", "LRecordField", "SAssign", "SSeq", "SIf", "SWhile", "SFor", "SMatch", "SReturn",
                    "SBarrier", "SWarpBarrier", "SExpr", "SEmpty", "SLet", "SLetMut", "SPragma", "SMemFence", "SBlock",
                    "SNative", "DParam", "DLocal", "DShared", "PConstr", "PWild"]
    assert [c for c in constructors if not re.search(r"\b" + c + r"\b", ml)] == []


def test_the_forms_the_ocaml_unit_test_expects_are_forms_the_native_reader_takes():
    """ocaml/sarek-hip/test/test_sarek_ir_hip.ml pins the text Sarek_ir_hip prints per IR constructor.  No compiler
    here can run it, so the other half of the contract is checked from this side: every expected string of that file
    goes through the library's reader and lowering inside a kernel."""
    from spoc_amd import hip
    ml = open(os.path.join(OCAML, "test", "test_sarek_ir_hip.ml")).read()

    def unescape(s):
        s = re.sub(r"\\\n\s*", "", s)                     # OCaml's line continuation inside a string
        return s.replace('\\"', '"').replace("\\\\", "\\")

    def table(name):
        body = re.search(r"let " + name + r" =\n(.*?)\n\n", ml, flags=re.S).group(1)
        return [unescape(s) for s in re.findall(r'"(\((?:[^"\\]|\\.)*)"\)', body)]

    def kernel(params="", body="(empty)"):
        return f"(kernel k (params{params}) (locals) (body {body}) (native_fn true))"

    types, consts = table("types"), table("constants_and_variables")
    exprs, stmts = table("expressions"), table("statements")
    assert (len(types), len(consts), len(exprs), len(stmts)) == (6, 7, 16, 18)
    for t in types:
        hip.generate_source(kernel(params=f" (param (var p 9 {t}))"))
    for e in consts + exprs:
        if e.startswith("(newarray"):                     # an array is created as the value of a let only
            hip.generate_source(kernel(body=f"(let (var tile 9 (array f32 shared)) {e} (empty))"))
        else:
            hip.generate_source(kernel(body=f"(expr {e})"))
    for s in stmts:
        hip.generate_source(kernel(body=s))
    whole = unescape(re.search(r'"(\(kernel sarek_kern (?:[^"\\]|\\.)*)"', ml, flags=re.S).group(1))
    src = hip.generate_source(whole)
    assert "void sarek_kern(float* __restrict__ a, int sarek_a_length, int n)" in src and "} point;" in src
    bare = re.search(r'"(\(intr \(Gpu\) [a-z_]+\))"', ml).group(1)
    # a name neither side knows goes out as a call of that name, for the device compiler to judge
    assert "no_such_intrinsic_for_this_test()" in hip.generate_source(kernel(body=f"(expr {bare})"))


def test_the_ocaml_test_directory_builds_against_the_plugin_library():
    dune = open(os.path.join(OCAML, "test", "dune")).read()
    tests = re.findall(r"\(name (\w+)\)", dune)
    assert sorted(tests) == ["test_hip_error", "test_sarek_ir_hip"]
    for t in tests:
        assert os.path.exists(os.path.join(OCAML, "test", t + ".ml")) and f"(modules {t})" in dune
    assert dune.count("sarek_hip") >= 2                   # the plugin library's dune name (ocaml/sarek-hip/dune)
    # every Hip_error constructor the error test builds is one the shared functor provides and the veneer raises
    # or could raise (spoc/framework/Backend_error.ml:291-347)
    err = open(os.path.join(OCAML, "test", "test_hip_error.ml")).read()
    functor = {"unknown_intrinsic", "invalid_arg_count", "unsupported_construct", "type_error", "invalid_memory_space",
               "unsupported_type", "no_device_selected", "device_not_found", "compilation_failed", "module_load_failed",
               "kernel_launch_failed", "memory_allocation_failed", "memory_copy_failed", "context_error",
               "synchronization_failed", "unsupported_source_lang", "backend_unavailable", "library_not_found",
               "initialization_failed", "feature_not_supported", "to_string", "raise_error", "with_default", "to_result",
               "Hip_error"}
    used = set(re.findall(r"Hip_error\.(\w+)", err))
    assert used and used <= functor, used - functor
