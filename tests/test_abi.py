"""The C-ABI library loads and exports every symbol include/sarek_hip.h declares.
No compute call is made here (this file runs without a GPU)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "sarek_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sarek_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(hip):
    names = declared_symbols()
    assert len(names) >= 45
    raw = ctypes.CDLL(hip.LIB_PATH)
    missing = [n for n in names if not hasattr(raw, n)]
    assert missing == []


def test_python_binding_covers_the_header(hip):
    assert sorted(hip.SYMBOLS) == declared_symbols()


def test_abi_version_and_status_names(hip):
    import __graft_entry__ as entry
    assert hip.lib.sarek_hip_abi_version() == entry.header_abi_version() >= 2
    entry.check_abi_version()       # the check build() ends with: it follows the header, not a literal
    assert hip.lib.sarek_hip_status_name(0) == b"SAREK_HIP_OK"
    assert hip.lib.sarek_hip_status_name(-2) == b"SAREK_HIP_E_UNSUPPORTED"
    assert hip.lib.sarek_hip_status_name(-5) == b"SAREK_HIP_E_WORKSPACE"


def test_backend_identity_and_intrinsic_registry(hip):
    """BACKEND.name / version / execution_model and BACKEND.Intrinsics (Framework_sig.ml:107-143,285,314):
    the lookups of sarek/framework/test/test_framework_integration.ml:190-207 against this backend."""
    import ctypes as C
    assert hip.lib.sarek_hip_backend_name() == b"HIP" and hip.lib.sarek_hip_execution_model() == 0      # JIT
    v = [C.c_int(-1) for _ in range(3)]
    hip.check(hip.lib.sarek_hip_backend_version(*[C.byref(x) for x in v]))
    assert [x.value for x in v] == [1, 0, 0]

    def find(name):
        buf, conv, found = C.create_string_buffer(128), C.c_int(-1), C.c_int(-1)
        hip.check(hip.lib.sarek_hip_intrinsic_find(name.encode(), buf, 128, C.byref(conv), C.byref(found)))
        return (buf.value.decode(), conv.value) if found.value else None

    def names():
        need = C.c_size_t(0)
        assert hip.lib.sarek_hip_intrinsic_list(None, 0, C.byref(need)) == hip.E_BUFFER_TOO_SMALL
        buf = C.create_string_buffer(need.value)
        hip.check(hip.lib.sarek_hip_intrinsic_list(buf, need.value, None))
        return buf.value.decode().split()
    UNIFORM, DIVERGENT, SYNC = 0, 1, 2
    assert find("thread_id_x") == ("threadIdx.x", DIVERGENT) and find("block_dim_z") == ("blockDim.z", UNIFORM)
    assert find("global_thread_id") == ("(threadIdx.x + blockIdx.x * blockDim.x)", DIVERGENT)
    assert find("block_barrier") == ("__syncthreads()", SYNC) and find("memory_fence") == ("__threadfence()", UNIFORM)
    assert find("warp_barrier")[1] == SYNC and "wave" in find("warp_barrier")[0]
    assert find("no_such_intrinsic") is None
    before = names()
    assert before == sorted(before) and len(before) >= 13 and "block_id_y" in before
    hip.check(hip.lib.sarek_hip_intrinsic_register(b"test_thread_id", b"threadIdx.x", DIVERGENT))
    hip.check(hip.lib.sarek_hip_intrinsic_register(b"test_thread_id", b"__lane_id()", DIVERGENT))       # replaces
    assert find("test_thread_id") == ("__lane_id()", DIVERGENT) and names().count("test_thread_id") == 1
    assert hip.lib.sarek_hip_intrinsic_register(b"x", b"y", 7) == hip.E_INVALID_ARG
    assert hip.lib.sarek_hip_intrinsic_register(b"", b"y", 0) == hip.E_INVALID_ARG
    small = C.create_string_buffer(4)
    found = C.c_int(0)
    assert hip.lib.sarek_hip_intrinsic_find(b"block_barrier", small, 4, None, C.byref(found)) == hip.E_BUFFER_TOO_SMALL


def test_is_available_never_raises(hip):
    # Framework_registry wraps is_available in try (sarek/framework/Framework_registry.ml:77-87)
    assert hip.lib.sarek_hip_is_available() in (0, 1)


def test_argument_validation_needs_no_gpu(hip):
    # invalid arguments are rejected before any HIP call is made
    assert hip.lib.sarek_hip_gemm_f32(None, None, None, 0, 4, 4, None) == hip.E_INVALID_ARG
    assert b"positive" in hip.lib.sarek_hip_last_error()
    assert hip.lib.sarek_hip_triad_f32(None, None, None, 3.0, -1, None) == hip.E_INVALID_ARG
    assert hip.lib.sarek_hip_triad_sum_f32(None, None, None, 3.0, 8, None, 0, None, None) == hip.E_INVALID_ARG
    blk = (ctypes.c_int * 3)(16, 16, 1)
    # unsupported source languages, error text in the reference's wording
    # (sarek-cuda/Cuda_plugin.ml:211-220)
    for lang, word in ((hip.LANG_OPENCL, b"OpenCL_Source"), (hip.LANG_PTX, b"PTX"),
                       (hip.LANG_SPIRV, b"SPIR_V"), (hip.LANG_GLSL, b"GLSL_Source")):
        rc = hip.lib.sarek_hip_run_source(b"x", lang, b"k", blk, blk, 0, None, 0)
        assert rc == hip.E_UNSUPPORTED
        assert word in hip.lib.sarek_hip_last_error()
    assert hip.lib.sarek_hip_mem_free(None) == 0
    assert hip.lib.sarek_hip_triad_sum_workspace_floats(1 << 28) >= 1


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    import importlib
    from spoc_amd import hip as real
    monkeypatch.setattr(real, "LIB_PATH", str(tmp_path / "nope.so"))
    try:
        real._load()
    except ImportError as e:
        assert "no CPU fallback" in str(e) or "not built" in str(e)
    else:
        raise AssertionError("loading a missing library must raise")
    importlib.reload(real)


C_CLIENT = r'''
#include <stdio.h>
#include <string.h>
#include "sarek_hip.h"
int main(void) {
  char key[33], dir[4096];
  int64_t stats[4];
  if (sarek_hip_abi_version() <= 0) return 1;
  if (sarek_hip_cache_compute_key("Device1", "1.0", "kernel code", key) != SAREK_HIP_OK) return 2;
  if (strlen(key) != 32) return 3;
  if (sarek_hip_cache_get_stats(stats) != SAREK_HIP_OK) return 4;
  if (sarek_hip_gemm_f32(NULL, NULL, NULL, 1, 1, 1, NULL) != SAREK_HIP_E_INVALID_ARG) return 5;
  if (strstr(sarek_hip_last_error(), "NULL") == NULL) return 6;
  if (sarek_hip_set_tunable(NULL, 1) != SAREK_HIP_E_INVALID_ARG) return 7;
  (void)dir;
  printf("%s\n", key);
  return 0;
}
'''


def test_header_is_c_and_a_c_client_links(hip, tmp_path):
    """include/sarek_hip.h is the boundary a C (or ctypes / cgo-style) client binds: it must
    compile as plain C99 with warnings on, and the library must link from C."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = tmp_path / "client.c"
    src.write_text(C_CLIENT)
    exe = tmp_path / "client"
    libdir = os.path.join(root, "spoc_amd")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.join(root, "include"),
                    str(src), "-o", str(exe), "-L", libdir, "-lsarek_hip", f"-Wl,-rpath,{libdir}",
                    "-Wl,-rpath,/opt/rocm/lib"], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.strip()
    import hashlib
    assert out == hashlib.md5(b"Device11.0kernel code").hexdigest()


def header_device_info_fields():
    """(name, C type text) of every member of sarek_hip_device_info, in order, from the header."""
    text = open(os.path.join(ROOT, "include", "sarek_hip.h")).read()
    body = re.search(r"typedef struct \{(.*?)\} sarek_hip_device_info;", text, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        ctype, names = decl.split(None, 1)
        for name in names.split(","):
            m = re.fullmatch(r"\s*(\w+)\s*(?:\[(\d+)\])?\s*", name)
            fields.append((m.group(1), ctype, int(m.group(2)) if m.group(2) else None))
    return fields


def test_device_info_layout_agrees_between_header_and_python(hip):
    """sarek_hip_device_get_info fills the whole struct: the Python binding must declare every member, in the
    header's order."""
    fields = header_device_info_fields()
    assert [f[0] for f in fields][-1] == "max_registers_per_block"
    assert [name for name, _ in hip.DeviceInfo._fields_] == [f[0] for f in fields]
    assert hip.lib.sarek_hip_device_info_size() == ctypes.sizeof(hip.DeviceInfo)

    # the OCaml stub's member list is checked against the same header in tests/test_ocaml_veneer.py


def test_device_report_never_needs_a_gpu(hip):
    """tools/device_info.ml:45-93: banner first; with no device the tool says so and exits 1."""
    text, count = hip.device_report()
    lines = text.split("\n")
    assert lines[0] == "=" * 70 and lines[1] == "SAREK Device Information Utility" and lines[3] == "=" * 70
    if count == 0:
        assert "No devices found" in text and "Found" not in text
    need = ctypes.c_size_t(0)
    small = ctypes.create_string_buffer(8)
    assert hip.lib.sarek_hip_device_report(small, 8, ctypes.byref(need), None) == hip.E_BUFFER_TOO_SMALL
    assert need.value == len(text.encode()) + 1


def test_library_kernel_texts_need_no_gpu(hip):
    """The texts a caller hands to Execute.run_source: complete HIP sources, tag first, found by name."""
    names = hip.library_kernel_names()
    assert names == ["gemm_bf16", "gemm_f16", "gemm_f16_bias_relu_rowsum", "triad_sum_f32"]
    for name in names:
        src, entry = hip.library_kernel(name)
        assert src.splitlines()[0] == "// sarek-hip-specialise: " + name
        assert f'extern "C" __global__ void {entry}(' in src and "Launch:" in src
        assert src.count("{") == src.count("}")
    need = ctypes.c_size_t(0)
    small = ctypes.create_string_buffer(16)
    assert hip.lib.sarek_hip_library_kernel_source(b"gemm_bf16", small, 16, ctypes.byref(need), None, 0) == hip.E_BUFFER_TOO_SMALL
    assert need.value > 200
    assert hip.lib.sarek_hip_library_kernel_source(b"no_such_kernel", None, 0, None, None, 0) == hip.E_INVALID_ARG
    assert b"no_such_kernel" in hip.lib.sarek_hip_last_error()
    assert hip.lib.sarek_hip_library_kernel_source(None, None, 0, None, None, 0) == hip.E_INVALID_ARG


def test_sequence_entry_points_validate_before_touching_a_device(hip):
    made, done = ctypes.c_int(7), ctypes.c_int(7)
    assert hip.lib.sarek_hip_run_sources(None, 0, ctypes.byref(made), ctypes.byref(done)) == 0
    assert (made.value, done.value) == (0, 0) and hip.lib.sarek_hip_last_run_path() == b"none"
    assert hip.lib.sarek_hip_run_sources(None, 2, None, None) == hip.E_INVALID_ARG
    assert hip.lib.sarek_hip_run_sources(None, -1, None, None) == hip.E_INVALID_ARG
    assert hip.lib.sarek_hip_execute_run_pipeline(None, 1, None) == hip.E_INVALID_ARG
    stage = (hip.PipelineStage * 1)()
    assert hip.lib.sarek_hip_execute_run_pipeline(stage, 1, None) == hip.E_INVALID_ARG      # NULL IR text
    assert b"stage 0" in hip.lib.sarek_hip_last_error()
    x = ctypes.c_double(0)
    assert hip.lib.sarek_hip_triad_block256_sum_f32(None, None, None, 3.0, -1, None, None) == hip.E_INVALID_ARG
    assert hip.lib.sarek_hip_triad_block256_sum_f32(None, None, None, 3.0, 0, None, None) == 0
    assert hip.lib.sarek_hip_triad_sum_f32_static(None, None, None, 3.0, 8, ctypes.byref(x), None) == hip.E_INVALID_ARG
    assert hip.lib.sarek_hip_triad_sum_f32_static(None, None, None, 3.0, (1 << 31) + 1, ctypes.byref(x), None) == hip.E_INVALID_ARG


def test_bench_refuses_more_than_one_gpu_without_touching_one():
    """bench.py measures one GPU; asked for more it says so and exits before it loads anything."""
    import subprocess
    import sys
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert run.returncode == 2 and "one GPU" in run.stderr and run.stdout == ""
