"""Four host threads, each with a stream of its own, launching through the library at once: 16-bit GEMMs that split K
(per-stream partial planes), the fused epilogue (per-stream row-sum planes), long folds (per-stream stages), element-wise
kernels through Execute.run_vectors (the rebuilt kernels' cached handles) and the triad / block-sum pipeline.  Every
result must be the one the same call gives alone.  ctypes releases the interpreter lock during a call, so the library's
own locks and per-stream resources are what keeps the threads apart."""
import threading

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_four_threads_on_four_streams(hip, torch_cuda):
    import sys
    import os
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from map_kernels import MAPS
    from spoc_amd import reference_kernels as rk
    from spoc_amd import sarek
    torch = torch_cuda
    sarek.Device.init()
    E, V = sarek.Execute, sarek.Vector

    def work(t, out):
        """One thread's share; `out` collects (name, tensor or array) pairs."""
        g = torch.Generator(device="cuda")
        g.manual_seed(100 + t)
        a = (torch.randn(256, 4096, device="cuda", generator=g) * 0.05).bfloat16()
        b = (torch.randn(4096, 256, device="cuda", generator=g) * 0.05).bfloat16()
        bias = torch.rand(1024, device="cuda", generator=g) * 0.2 - 0.1
        ea = (torch.randn(300, 128, device="cuda", generator=g) * 0.05).half()
        eb = (torch.randn(128, 1024, device="cuda", generator=g) * 0.05).half()
        parts = torch.rand((1 << 18) + 1000 * t, device="cuda", generator=g) * 100
        x = np.random.default_rng(t).standard_normal(50000 + t).astype(np.float32)
        for it in range(12):
            out.append((f"gemm{it}", hip.gemm_bf16(a, b).clone()))                  # K split over idle CUs
            y, rs = hip.gemm_f16_bias_relu_rowsum(ea, eb, bias)
            out.append((f"rowsum{it}", rs.clone()))
            out.append((f"fold{it}", hip.fold_partials(parts).clone()))
            n = x.size
            res = V.create(V.float32, n)
            E.run_vectors(MAPS["scale"](), [E.Vec(V.of_array(x)), E.Vec(res), E.Float32(1.5 + t), E.Int32(n)],
                          (256, 1, 1), ((n + 255) // 256, 1, 1))
            out.append((f"map{it}", res.to_array().copy()))
            va, sums = V.create(V.float32, n), V.create(V.float32, (n + 255) // 256)
            shape = ((256, 1, 1), ((n + 255) // 256, 1, 1))
            E.run_pipeline([(rk.stream_triad(), [E.Vec(va), E.Vec(V.of_array(x)), E.Vec(V.of_array(x[::-1].copy())),
                                                 E.Float32(3.0), E.Int32(n)]) + shape,
                            (rk.tree(False), [E.Vec(va), E.Vec(sums), E.Int32(n)]) + shape])
            out.append((f"sums{it}", sums.to_array().copy()))
        torch.cuda.synchronize()

    assert hip.gemm16_k_splits(256, 256, 4096) > 1
    # each thread's share runs on one stream both times: what a stream's calls may use (a block for K-split partials,
    # a stage for long folds) is the same alone and together, however many streams the process has seen before
    streams = [torch.cuda.Stream() for _ in range(4)]
    assert len({st.cuda_stream for st in streams}) == 4
    alone = []
    for t in range(4):
        alone.append([])
        with torch.cuda.stream(streams[t]):
            work(t, alone[t])
    together, errors = [[] for _ in range(4)], []

    def threaded(t):
        try:
            with torch.cuda.stream(streams[t]):
                work(t, together[t])
        except Exception as e:              # noqa: BLE001 -- reported by the main thread
            errors.append((t, repr(e)))

    threads = [threading.Thread(target=threaded, args=(t,)) for t in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    torch.cuda.synchronize()
    assert errors == []
    for t in range(4):
        assert len(together[t]) == len(alone[t])
        for (name, got), (_, want) in zip(together[t], alone[t]):
            same = np.array_equal(got, want) if isinstance(got, np.ndarray) else torch.equal(got, want)
            assert same, (t, name)


def test_long_folds_on_more_streams_than_the_library_has_stages(hip, torch_cuda):
    """Long folds keep their per-workgroup sums in one of sixteen stages a device holds, one per stream; a stream
    that comes when all are taken folds with one workgroup.  Twenty-four streams, seven lengths (one, two, four and
    more loads per thread and piece, unaligned ones among them): every sum is, bit for bit, the one the default
    stream gives."""
    torch = torch_cuda
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    streams = {torch.cuda.Stream().cuda_stream: None for _ in range(64)}
    streams = [torch.cuda.ExternalStream(s) for s in streams][:24]
    assert len(streams) == 24
    for n, offset in (((1 << 17) + 0, 0), ((1 << 20) - 3, 0), ((1 << 19) + 5, 1), ((1 << 21) - 77, 0), ((1 << 22) - 3, 0),
                      ((1 << 22) + 4096, 0), ((1 << 21) + 1, 3)):
        x = (torch.rand(n + offset, device="cuda", generator=g) * 100)[offset:]
        want = torch.zeros(1, dtype=torch.float64, device="cuda")
        hip.check(hip.lib.sarek_hip_fold_partials_f64(x.data_ptr(), n, want.data_ptr(), None))
        torch.cuda.synchronize()
        assert abs(want.item() - float(x.cpu().numpy().astype("float64").sum())) <= 1e-12 * want.item()
        got = torch.zeros(len(streams), dtype=torch.float64, device="cuda")
        for k, st in enumerate(streams):
            hip.check(hip.lib.sarek_hip_fold_partials_f64(x.data_ptr(), n, got[k:].data_ptr(), st.cuda_stream))
        torch.cuda.synchronize()
        assert bool((got == want).all()), (n, offset, got.tolist(), want.item())
