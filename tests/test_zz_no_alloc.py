"""sarek_hip_triad_sum_f32_static, the entry point that allocates nothing: called through the C ABI
with buffers made beforehand, checked bit for bit against sarek_hip_triad_sum_f32 (same kernels,
caller workspace) and against the oracle, on two calls in a row, the second with a smaller input
(the built-in partials array still holds the first call's values then)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def ptr(t):
    return C.c_void_p(t.data_ptr())


def test_static_triad_sum_matches_the_workspace_entry_point_twice_in_a_row(hip, oracle, torch_cuda):
    torch = torch_cuda
    lib = hip.lib
    sizes = [(1 << 22) + 4099, 70001]       # second call: smaller, ragged, fewer workgroups
    nmax = max(sizes)
    # every buffer exists before the calls under test
    b_all = torch.from_numpy(oracle.fill_uniform(nmax, seed=0xB)).cuda()
    c_all = torch.from_numpy(oracle.fill_uniform(nmax, seed=0xC)).cuda()
    a_static = torch.empty(nmax, dtype=torch.float32, device="cuda")
    a_ws = torch.empty(nmax, dtype=torch.float32, device="cuda")
    sum_static = torch.zeros(1, dtype=torch.float64, device="cuda")
    sum_ws = torch.zeros(1, dtype=torch.float64, device="cuda")
    partials = torch.empty(int(lib.sarek_hip_triad_sum_workspace_floats(nmax)), dtype=torch.float32, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()

    for n in sizes:
        a_static.fill_(-1.0)
        a_ws.fill_(-2.0)
        before = torch.cuda.memory_allocated()
        hip.check(lib.sarek_hip_triad_sum_f32_static(ptr(a_static), ptr(b_all), ptr(c_all), 3.0, n,
                                                     ptr(sum_static), stream))
        assert torch.cuda.memory_allocated() == before
        hip.check(lib.sarek_hip_triad_sum_f32(ptr(a_ws), ptr(b_all), ptr(c_all), 3.0, n, ptr(partials),
                                              partials.numel(), ptr(sum_ws), stream))
        torch.cuda.synchronize()
        got_a, want_a = a_static[:n].cpu().numpy(), a_ws[:n].cpu().numpy()
        assert np.array_equal(got_a, want_a)
        assert float(a_static[n:].min().item()) == -1.0 if n < nmax else True     # nothing written past n
        assert sum_static.item() == sum_ws.item()                                  # same kernels, same order
        a_ref, _, sum_ref = oracle.triad_sum(b_all[:n].cpu().numpy(), c_all[:n].cpu().numpy(), 3.0)
        assert np.array_equal(got_a, a_ref)
        assert abs(sum_static.item() - sum_ref) <= 1e-5 * abs(sum_ref)

    # empty input: the sum is set to zero, nothing else is touched
    hip.check(lib.sarek_hip_triad_sum_f32_static(None, None, None, 3.0, 0, ptr(sum_static), stream))
    torch.cuda.synchronize()
    assert sum_static.item() == 0.0


def test_static_triad_sum_refuses_what_its_array_cannot_serve(hip, torch_cuda):
    torch = torch_cuda
    lib = hip.lib
    limit = int(lib.sarek_hip_triad_sum_static_max_n())
    assert limit == 1 << 31
    x = torch.zeros(16, dtype=torch.float32, device="cuda")
    out = torch.full((1,), 7.0, dtype=torch.float64, device="cuda")
    # refused on the length alone, before any launch: the small buffers are never touched
    rc = lib.sarek_hip_triad_sum_f32_static(ptr(x), ptr(x), ptr(x), 3.0, limit + 1, ptr(out), None)
    assert rc == hip.E_WORKSPACE and b"at most" in lib.sarek_hip_last_error()
    assert lib.sarek_hip_triad_sum_f32_static(ptr(x), ptr(x), ptr(x), 3.0, -1, ptr(out), None) == hip.E_INVALID_ARG
    assert lib.sarek_hip_triad_sum_f32_static(ptr(x), ptr(x), ptr(x), 3.0, 4, None, None) == hip.E_INVALID_ARG
    torch.cuda.synchronize()
    assert out.item() == 7.0
