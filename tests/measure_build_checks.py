"""Checks of libsarek_hip_measure.so, run as a script by tests/test_gpu_gemm.py with SAREK_HIP_MEASURE_BUILD=1 in a
process of its own (pytest does not collect this file): the measurement build is the product's sources plus the kernel
variants of the ablation studies, so its default kernel must give the product's results, its extra kernels must agree
with the oracle where they compute the product (the 32 x 32 x 16 pipeline in its ring and wave shapes) and stay
within the operands' bounds where they do not (the variants that leave parts of the K loop out)."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import torch  # noqa: E402

import oracle  # noqa: E402
from spoc_amd import hip  # noqa: E402


def dev(x):
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def normal16(shape, seed):
    rng = np.random.default_rng(seed)
    return oracle.round_bf16(rng.normal(0, 0.02, shape).astype(np.float32))


def main():
    assert hip.MEASURE_BUILD and hip.lib.sarek_hip_is_measurement_build() == 1
    torch.cuda.set_device(0)

    # every ring / wave shape of the 32 x 32 x 16 kernel and the 16 x 16 x 32 kernel against the oracle
    for (m, n, k) in [(300, 520, 64), (257, 136, 192), (512, 768, 448), (70, 1032, 1216)]:
        a, b = normal16((m, k), m), normal16((k, n), n)
        ref = oracle.gemm(a, b)
        da, db = dev(a).bfloat16(), dev(b).bfloat16()
        for ring, tj, mfma in [(0, 2, 16), (0, 2, 32), (0, 4, 32), (4, 2, 32), (4, 4, 32), (2, 2, 32), (2, 4, 32)]:
            hip.set_tunable("gemm16.ring", ring)
            hip.set_tunable("gemm16.tj", tj)
            hip.set_tunable("gemm16.mfma", mfma)
            hip.set_tunable("gemm16.tile", 256)
            try:
                c = hip.gemm_bf16(da, db).cpu().numpy()
            finally:
                hip.set_tunable("gemm16.ring", 0)
                hip.set_tunable("gemm16.tj", 2)
                hip.set_tunable("gemm16.mfma", 16)
                hip.set_tunable("gemm16.tile", 0)
            assert np.abs(c - ref).max() / np.abs(ref).max() < 1e-4, (m, n, k, ring, tj, mfma)
    print("ring shapes ok", flush=True)

    # the 4-wave kernel (128 x 128 per wave, asm MFMAs on AGPR accumulators): the 8-wave kernel's bits
    for (m, n, k) in [(256, 256, 64), (512, 768, 448), (300, 520, 192), (1024, 1024, 1216), (70, 1032, 128)]:
        a, b = normal16((m, k), m + 1), normal16((k, n), n + 1)
        da, db = dev(a).bfloat16(), dev(b).bfloat16()
        hip.set_tunable("gemm16.tile", 256)
        try:
            ref = hip.gemm_bf16(da, db)
            ref16 = hip.gemm_f16(da.half(), db.half())
            hip.set_tunable("gemm16.waves", 4)
            got = hip.gemm_bf16(da, db)
            got16 = hip.gemm_f16(da.half(), db.half())
        finally:
            hip.set_tunable("gemm16.waves", 8)
            hip.set_tunable("gemm16.tile", 0)
        assert torch.equal(got, ref) and torch.equal(got16, ref16), (m, n, k)
    print("4-wave kernel ok", flush=True)

    # one barrier per K = 64 instead of per K = 32 (a deeper B ring): the 8-wave kernel's bits, run after run
    for (m, n, k) in [(256, 256, 64), (256, 256, 192), (512, 768, 448), (300, 520, 256), (1024, 1024, 1216)]:
        a, b = normal16((m, k), m + 2), normal16((k, n), n + 2)
        da, db = dev(a).bfloat16(), dev(b).bfloat16()
        bias = dev(np.linspace(-0.1, 0.1, n, dtype=np.float32))
        hip.set_tunable("gemm16.tile", 256)
        try:
            ref, ref16 = hip.gemm_bf16(da, db), hip.gemm_f16(da.half(), db.half())
            y_ref, rs_ref = hip.gemm_f16_bias_relu_rowsum(da.half(), db.half(), bias)
            hip.set_tunable("gemm16.barriers", 1)
            for _ in range(3):
                assert torch.equal(hip.gemm_bf16(da, db), ref) and torch.equal(hip.gemm_f16(da.half(), db.half()), ref16)
            y, rs = hip.gemm_f16_bias_relu_rowsum(da.half(), db.half(), bias)
            assert torch.equal(y, y_ref) and torch.equal(rs, rs_ref), (m, n, k)
        finally:
            hip.set_tunable("gemm16.barriers", 2)
            hip.set_tunable("gemm16.tile", 0)
    print("half-barrier kernel ok", flush=True)

    # the ablated variants: wrong by construction, but within bounds; other kernels refuse the knob
    m, n, k = 512, 768, 512
    torch.manual_seed(7)
    a = (torch.randn(m, k, device="cuda") * 0.1).bfloat16()
    b = (torch.randn(k, n, device="cuda") * 0.1).bfloat16()
    good = hip.gemm_bf16(a, b)
    try:
        for mfma, variants in ((16, (1, 2, 3)), (32, (1, 2, 3, 4))):
            hip.set_tunable("gemm16.mfma", mfma)
            for v in variants:
                hip.set_tunable("gemm16.ablate", v)
                c = hip.gemm_bf16(a, b)
                torch.cuda.synchronize()
                assert torch.isfinite(c).all(), (mfma, v)
        hip.set_tunable("gemm16.ablate", 8)
        untouched = torch.full((m, n), 7.0, device="cuda")
        hip.gemm_bf16(a, b, out=untouched)
        torch.cuda.synchronize()
        assert bool((untouched == 7.0).all())
        for mfma in (16, 32):
            hip.set_tunable("gemm16.mfma", mfma)
            hip.set_tunable("gemm16.ablate", 1)
            try:
                hip.gemm_f16(a.half(), b.half())
                raise AssertionError("fp16 took an ablated kernel")
            except hip.SarekHipError as e:
                assert e.status == hip.E_UNSUPPORTED
            hip.set_tunable("gemm16.ablate", 5)
            try:
                hip.gemm_bf16(a, b)
                raise AssertionError("ablate=5 was accepted")
            except hip.SarekHipError:
                pass
    finally:
        hip.set_tunable("gemm16.ablate", 0)
        hip.set_tunable("gemm16.mfma", 16)
    assert torch.equal(hip.gemm_bf16(a, b), good)
    print("ablated variants ok", flush=True)

    # the in-kernel clock probe: one (cycles, ticks) pair per workgroup, a plausible clock, nothing once it is off
    m = n = 1024
    k = 512
    a = torch.randn(m, k, device="cuda").to(torch.bfloat16)
    b = torch.randn(k, n, device="cuda").to(torch.bfloat16)
    with hip.clock_probe(workgroups=64) as probe:
        hip.gemm_bf16(a, b)                      # 64 workgroups of 128 x 128
        assert hip.gemm16_tile(m, n, k) == 128 and len(probe.pairs()) == 64
        assert 500 < probe.mhz() < 2600
        probe.buf.zero_()
        hip.set_tunable("gemm16.tile", 256)
        try:
            hip.gemm_bf16(a, b)                  # 16 workgroups of 256 x 256
        finally:
            hip.set_tunable("gemm16.tile", 0)
        assert len(probe.pairs()) == 16 and 500 < probe.mhz() < 2600
        probe.buf.zero_()
        hip.gemm_bf16(torch.zeros(4096, 64, device="cuda", dtype=torch.bfloat16),
                      torch.zeros(64, 8192, device="cuda", dtype=torch.bfloat16))   # 512 workgroups > 64 pairs
        assert len(probe.pairs()) == 0
    probe.buf.zero_()
    hip.gemm_bf16(a, b)
    assert len(probe.pairs()) == 0
    x = torch.randn(512, 256, device="cuda")
    with hip.clock_probe(workgroups=64) as probe:
        hip.gemm_f32(x, x[:256, :].contiguous())
        assert len(probe.pairs()) > 0 and 500 < probe.mhz() < 2600
    print("clock probe ok", flush=True)
    print("measurement build ok", flush=True)


if __name__ == "__main__":
    main()
