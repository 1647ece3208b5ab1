"""The library's host code (IR reader, HIP lowering, recogniser, fusion, Vector storage) built with
AddressSanitizer and UndefinedBehaviorSanitizer and driven over damaged IR texts and the Vector
module's storage functions.  No GPU is involved: the .hip files stay out of the build."""
import concurrent.futures
import glob
import os
import random
import re
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(ROOT, "spoc_amd", "csrc")
CLANG = "/opt/rocm/llvm/bin/clang++"


def damaged_texts(count, seed):
    from spoc_amd import reference_kernels as rk
    rng = random.Random(seed)
    texts = [open(f).read() for f in sorted(glob.glob(os.path.join(HERE, "golden", "ir", "*.ir")))]
    texts += [rk.histogram(), rk.nbody_accel(), rk.conv2d(), rk.inclusive_scan(), rk.stencil_2d()]
    # names bound again, loops with moving bounds, helper functions, int64, matches with payloads and variable patterns
    import ir_programs
    from test_ir_lowering import MATCH_AS_A_VALUE, MATCH_WITH_A_VARIABLE_PATTERN
    texts += [ir_programs.random_program(s)[0] for s in range(10)] + [MATCH_AS_A_VALUE, MATCH_WITH_A_VARIABLE_PATTERN]
    spare = ["i32", "f32", "(var x 1 i32)", "add", "read", "let", "seq", "(i32 0)", "shared", "vec", "-",
             "99999999999999999999", '"', "template", "match", "case", "record", "variant", "app", "for", "upto",
             "mut", "output", "a"]
    out = []
    for _ in range(count):
        t = rng.choice(texts)
        r = rng.random()
        if 0.2 <= r < 0.65:
            toks = re.findall(r'\(|\)|"[^"]*"|[^\s()]+', t)
            atoms = [k for k, x in enumerate(toks) if x not in "()"]
            for _ in range(rng.randint(1, 4)):
                a, b = rng.choice(atoms), rng.choice(atoms)
                toks[a] = toks[b] if rng.random() < 0.7 else rng.choice(spare)
            t = " ".join(toks)
        elif r >= 0.65:
            for _ in range(rng.randint(1, 3)):
                if not t:
                    break
                i = rng.randrange(len(t))
                j = min(len(t), i + rng.randint(1, 40))
                t = (t[:i] + t[j:], t[:i] + t[i:j] * 2 + t[j:], t[:i] + rng.choice(spare) + t[j:],
                     t[:i] + rng.choice(spare) + t[i:], t[:i])[rng.randint(0, 4)]
        out.append(t.replace("\0", ""))
    return out


def build_driver(tmp_path, sanitizers, name):
    """The driver and the library's host sources compiled and linked with -fsanitize=<sanitizers>."""
    sources = [os.path.join(HERE, "host_sanitizers", f) for f in ("driver.cpp", "kernel_stubs.cpp")]
    sources += [os.path.join(CSRC, f) for f in (
        "status.cpp", "backend_info.cpp", "tunables.cpp", "runtime.cpp", "transfer.cpp", "vector.cpp", "gpu_memory.cpp",
        "code_cache.cpp", "plugin.cpp", "library_kernels.cpp", "generate.cpp", "fusion_abi.cpp", "host/ir_text.cpp", "host/ir_hip.cpp",
        "host/specialise.cpp", "host/fusion.cpp", "host/map_fuse.cpp")]
    exe = str(tmp_path / name)
    flags = ["-std=c++20", "-O1", "-g", "-fsanitize=" + sanitizers, "-fno-omit-frame-pointer", "-D__HIP_PLATFORM_AMD__",
             "-I/opt/rocm/include", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC, "-w"]
    if "undefined" in sanitizers:
        flags.append("-fno-sanitize-recover=undefined")

    def compile_one(item):
        k, src = item
        obj = str(tmp_path / f"{name}_{k}.o")
        done = subprocess.run([CLANG, *flags, "-c", src, "-o", obj], capture_output=True, text=True)
        assert done.returncode == 0, done.stderr[-3000:]
        return obj
    with concurrent.futures.ThreadPoolExecutor(max_workers=8) as pool:      # the compiler processes do the work
        objects = list(pool.map(compile_one, enumerate(sources)))
    build = subprocess.run([CLANG, "-fsanitize=" + sanitizers, *objects, "-L/opt/rocm/lib", "-lamdhip64",
                            "-lhiprtc", "-lpthread", "-Wl,-rpath,/opt/rocm/lib", "-o", exe],
                           capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-3000:]
    return exe


@pytest.mark.skipif(not os.path.exists(CLANG), reason="no clang++ with sanitizer runtimes in this image")
def test_host_code_is_clean_under_asan_and_ubsan(tmp_path):
    exe = build_driver(tmp_path, "address,undefined", "host_asan")
    records = tmp_path / "records.bin"
    records.write_bytes("\0".join(damaged_texts(1500, seed=77)).encode())
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    run = subprocess.run([exe, str(records)], capture_output=True, text=True, env=env, timeout=600)
    assert run.returncode == 0, (run.stdout[-2000:], run.stderr[-4000:])
    assert "vector storage ok" in run.stdout and "records 1500" in run.stdout
    assert "ERROR: AddressSanitizer" not in run.stderr and "runtime error" not in run.stderr


@pytest.mark.skipif(not os.path.exists(CLANG), reason="no clang++ with sanitizer runtimes in this image")
def test_host_code_is_free_of_data_races_under_tsan(tmp_path):
    """Eight threads lower the same 150 texts (sound and damaged), rebuild map kernels, fuse, set and read tunables,
    count device memory, compute cache keys and work on vectors of their own, all at once, under ThreadSanitizer:
    the caches the lowering keeps between calls (tagged texts, rebuilt-kernel entries) and the library's counters must
    take that without a report."""
    exe = build_driver(tmp_path, "thread", "host_tsan")
    from spoc_amd import reference_kernels as rk
    import sys
    sys.path.insert(0, HERE)
    import map_kernels
    texts = [open(f).read() for f in sorted(glob.glob(os.path.join(HERE, "golden", "ir", "*.ir")))]
    texts += [rk.histogram(), rk.stencil_2d()] + [make() for make in map_kernels.MAPS.values()]
    texts += [make() for make in map_kernels.TREES.values()] + [make() for make in map_kernels.MAX_TREES.values()]
    texts += [map_kernels.random_map(seed)[0] for seed in range(20)] + damaged_texts(100, seed=5)
    records = tmp_path / "records_threads.bin"
    records.write_bytes("\0".join(texts).encode())
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=0:report_signal_unsafe=0")
    run = subprocess.run([exe, str(records), "threads"], capture_output=True, text=True, env=env, timeout=900)
    assert "WARNING: ThreadSanitizer" not in run.stderr, run.stderr[-6000:]
    assert run.returncode == 0 and "threads ok" in run.stdout, (run.stdout[-2000:], run.stderr[-4000:])
