"""Kernel fusion on IR text: the functions of sarek/sarek/Sarek_fusion.ml, by the same names
and with the same meaning, over the C ABI of libsarek_hip (the pass itself is native code).
Kernels, statements and expressions are the s-expression text sarek_hip_generate_source reads.
"""
import ctypes as C
import re
from collections import namedtuple

from . import hip

VERTICAL, REDUCTION, STENCIL, TRY, TRY_ALL = range(5)
Fuse, DontFuse, MaybeFuse = "Fuse", "DontFuse", "MaybeFuse"

FusionInfo = namedtuple("FusionInfo", "reads writes has_barriers has_atomics")     # Sarek_fusion.ml:25-30
FusionHint = namedtuple("FusionHint", "decision reason")                            # :1044
StencilFusionInfo = namedtuple("StencilFusionInfo",
                               "combined_radius producer_radius consumer_radius input_arrays")   # :821-826
ReductionLoop = namedtuple("ReductionLoop", "acc acc_id op array loop_var loop_var_id")


class FusionError(hip.SarekHipError):
    """Fusion_error.Fusion_error (sarek/sarek/Fusion_error.ml:28)."""


def _text(call, *head):
    """Calls an entry point whose last three parameters are (out, out_len, needed)."""
    needed = C.c_size_t(0)
    cap = 1 << 14
    while True:
        buf = C.create_string_buffer(cap)
        st = call(*head, buf, cap, C.byref(needed))
        if st == hip.E_BUFFER_TOO_SMALL and needed.value > cap:
            cap = needed.value
            continue
        hip.check(st)
        return buf.value.decode()


def _b(s):
    return s.encode()


def _split_top(text):
    """Top-level items of an s-expression list body."""
    items, depth, cur = [], 0, ""
    for ch in text:
        if ch == "(":
            depth += 1
        if ch == ")":
            depth -= 1
        if ch.isspace() and depth == 0:
            if cur:
                items.append(cur)
            cur = ""
        else:
            cur += ch
    if cur:
        items.append(cur)
    return items


def _patterns(section):
    """'(NAME pattern) (NAME pattern) ...' -> list of (name, pattern)."""
    out = []
    for item in _split_top(section):
        name, pat = item[1:-1].split(" ", 1)
        if pat.startswith("(one_to_one "):
            out.append((name, ("OneToOne", pat[len("(one_to_one "):-1])))
        elif pat.startswith("(stencil"):
            out.append((name, ("Stencil", [int(x) for x in pat[len("(stencil"):-1].split()])))
        elif pat.startswith("(reduction "):
            out.append((name, ("Reduction", pat[len("(reduction "):-1])))
        else:
            out.append((name, ("Gather" if pat == "gather" else "Unknown", None)))
    return out


def analyze(kernel):
    """Sarek_fusion.analyze (:340-354).  reads / writes: [(array, (kind, detail))] sorted by array,
    kind in OneToOne (detail = index expression text), Stencil (sorted offsets), Reduction
    (operator word), Gather, Unknown."""
    text = _text(hip.lib.sarek_hip_fusion_analyze, _b(kernel))
    m = re.fullmatch(r"\(info \(reads ?(.*)\) \(writes ?(.*)\) \(barriers (true|false)\) \(atomics (true|false)\)\)",
                     text, re.S)
    return FusionInfo(_patterns(m.group(1)), _patterns(m.group(2)), m.group(3) == "true", m.group(4) == "true")


def _can(producer, consumer, intermediate, mode):
    r = C.c_int(0)
    hip.check(hip.lib.sarek_hip_fusion_can_fuse(_b(producer), _b(consumer), _b(intermediate), mode, C.byref(r)))
    return bool(r.value)


def _fuse(producer, consumer, intermediate, mode):
    fused = C.c_int(0)
    text = _text(hip.lib.sarek_hip_fusion_fuse, _b(producer), _b(consumer), _b(intermediate), mode, C.byref(fused))
    return text if fused.value else None


def can_fuse(producer, consumer, intermediate): return _can(producer, consumer, intermediate, VERTICAL)
def fuse(producer, consumer, intermediate): return _fuse(producer, consumer, intermediate, VERTICAL)
def can_fuse_reduction(m, r, intermediate): return _can(m, r, intermediate, REDUCTION)
def fuse_reduction(m, r, intermediate): return _fuse(m, r, intermediate, REDUCTION)
def can_fuse_stencil(producer, consumer, intermediate): return _can(producer, consumer, intermediate, STENCIL)
def fuse_stencil(producer, consumer, intermediate): return _fuse(producer, consumer, intermediate, STENCIL)
def try_fuse(producer, consumer, intermediate): return _fuse(producer, consumer, intermediate, TRY)
def try_fuse_all(producer, consumer, intermediate): return _fuse(producer, consumer, intermediate, TRY_ALL)


def should_fuse(producer, consumer, intermediate):
    d = C.c_int(0)
    reason = C.create_string_buffer(128)
    hip.check(hip.lib.sarek_hip_fusion_should_fuse(_b(producer), _b(consumer), _b(intermediate), C.byref(d),
                                                   reason, len(reason)))
    return FusionHint((Fuse, DontFuse, MaybeFuse)[d.value], reason.value.decode())


def _pipeline(kernels, automatic):
    arr = (C.c_char_p * max(len(kernels), 1))(*[_b(k) for k in kernels])
    needed, rneeded = C.c_size_t(0), C.c_size_t(0)
    cap = rcap = 1 << 14
    while True:
        out, rep = C.create_string_buffer(cap), C.create_string_buffer(rcap)
        st = hip.lib.sarek_hip_fusion_pipeline(arr, len(kernels), automatic, out, cap, C.byref(needed), rep, rcap,
                                               C.byref(rneeded))
        if st == hip.E_BUFFER_TOO_SMALL and (needed.value > cap or rneeded.value > rcap):
            cap, rcap = max(cap, needed.value), max(rcap, rneeded.value)
            continue
        if st == hip.E_INVALID_ARG:
            raise FusionError(st, "invalid argument", hip.lib.sarek_hip_last_error().decode())
        hip.check(st)
        lines = rep.value.decode().splitlines()
        return (out.value.decode(), [l[len("eliminated "):] for l in lines if l.startswith("eliminated ")],
                [l[len("skipped "):] for l in lines if l.startswith("skipped ")])


def fuse_pipeline(kernels):
    """(fused kernel, eliminated arrays, latest first) — Sarek_fusion.fuse_pipeline (:570-598)."""
    k, eliminated, _ = _pipeline(kernels, 0)
    return k, eliminated


def auto_fuse_pipeline(kernels):
    """(fused kernel, eliminated arrays, skipped reasons) — Sarek_fusion.auto_fuse_pipeline (:1133-1165)."""
    return _pipeline(kernels, 1)


def analyze_pipeline(kernels):
    """The text Sarek_fusion.analyze_pipeline prints (:1180-1214)."""
    arr = (C.c_char_p * max(len(kernels), 1))(*[_b(k) for k in kernels])
    return _text(hip.lib.sarek_hip_fusion_analyze_pipeline, arr, len(kernels))


def analyze_stencil_fusion(producer, consumer, intermediate):
    found = C.c_int(0)
    radii = (C.c_int * 3)()
    names = _text(hip.lib.sarek_hip_fusion_stencil_info, _b(producer), _b(consumer), _b(intermediate),
                  C.byref(found), radii)
    return StencilFusionInfo(radii[0], radii[1], radii[2], names.split()) if found.value else None


def stencil_radius(offsets):
    """Sarek_fusion.stencil_radius (:779-780)."""
    return max([abs(o) for o in offsets], default=0)


def expr_equal(a, b):
    r = C.c_int(0)
    hip.check(hip.lib.sarek_hip_fusion_expr_equal(_b(a), _b(b), C.byref(r)))
    return bool(r.value)


def subst_array_read(arr, idx, replacement, expr):
    return _text(hip.lib.sarek_hip_fusion_subst_array_read, _b(arr), _b(idx), _b(replacement), _b(expr))


def detect_reduction_pattern(stmt):
    found = C.c_int(0)
    text = _text(hip.lib.sarek_hip_fusion_detect_reduction, _b(stmt), C.byref(found))
    if not found.value:
        return None
    _, acc, acc_id, op, array, loop_var, loop_id = text[1:-1].split()
    return ReductionLoop(acc, int(acc_id), op, array, loop_var, int(loop_id))


def is_reduction_kernel(kernel, arr):
    found = C.c_int(0)
    op = C.create_string_buffer(8)
    hip.check(hip.lib.sarek_hip_fusion_is_reduction_kernel(_b(kernel), _b(arr), C.byref(found), op))
    return op.value.decode() if found.value else None
