"""Random walks through Vector / Transfer / Execute against a model of the reference's state machine.

The model below is written from the reference's text, operation by operation, and knows nothing of the library:

  Vector.get / set / fill / blit / copy / sub_vector      sarek/core/Vector.ml:80-133, 220-250, 500-517
  ensure_cpu_sync and the callback Transfer registers      sarek/core/Vector_transfer.ml:46-53, Transfer.ml:452-464
  Transfer.to_device / to_cpu ?force / sync / free_all     sarek/core/Transfer.ml:228-348, 371-381
  Execute.run_vectors: upload the arguments, launch,
  mark Both vectors Stale_CPU                              sarek/sarek/Execute.ml:188-190, 321-335, 520-543

A vector is a host array (a sub-vector's is a view of its parent's), a device array or none, a location and its
auto-sync flag; the kernel of a launch is v[i] <- 2 v[i] + 1 on the device copy.  After every step of a walk the
library's vector must show the model's location, its host block the model's host array (read raw, behind the
library's back) and its device buffer the model's device array -- including the reference's corners: a host write into
a Stale_CPU vector is not tracked and is overwritten by the next download, a write into a GPU-only vector marks it
Stale_GPU although the host copy was never fetched, a sub-vector writes through to its parent's host block without
touching the parent's location."""
import ctypes as C
import os
import random

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

CPU, GPU, BOTH, STALE_CPU, STALE_GPU = "CPU", "GPU", "Both", "Stale_CPU", "Stale_GPU"


class Model:
    """One vector of the reference, as its source describes it."""
    auto_mode = True                                  # Transfer.auto_mode

    def __init__(self, host):
        self.host, self.device, self.location, self.auto_sync = host, None, CPU, True

    def ensure_cpu_sync(self):
        if self.auto_sync and self.location == STALE_CPU and Model.auto_mode:
            self.to_cpu()

    def host_write(self):                             # the tail of set / unsafe_set / fill
        if self.location in (BOTH, GPU):
            self.location = STALE_GPU

    def get(self, i):
        self.ensure_cpu_sync()
        return self.host[i]

    def set(self, i, x):
        self.host[i] = x
        self.host_write()

    def fill(self, x):
        self.host[:] = x
        self.host_write()

    def to_device(self):
        if self.location in (GPU, BOTH, STALE_CPU):
            return
        self.device = self.host.copy()
        self.location = BOTH

    def to_cpu(self, force=False):
        if self.location in (GPU, STALE_CPU) or (self.location == BOTH and force):
            self.host[:] = self.device
            self.location = BOTH

    def sync(self):
        if self.location in (GPU, STALE_CPU):
            self.to_cpu()
        elif self.location == STALE_GPU:
            self.to_device()

    def free_all_buffers(self):
        self.device, self.location = None, CPU

    def launch(self):
        self.to_device()
        self.device = self.device * np.float32(2) + np.float32(1)
        if self.location == BOTH:
            self.location = STALE_CPU


@pytest.fixture()
def sarek(hip, torch_cuda):
    from spoc_amd import sarek as s
    s.Device.init()
    yield s
    s.Transfer.set_auto(True)


def device_contents(hip, v):
    ptr = v.device_ptr
    if ptr is None:
        return None
    out = np.empty(v.length, np.float32)
    hip.check(hip.lib.sarek_hip_device_synchronize())
    hip.check(hip.lib.sarek_hip_memcpy_dtoh(C.c_void_p(out.ctypes.data), C.c_void_p(ptr), out.nbytes))
    return out


@pytest.mark.parametrize("seed", range(int(os.environ.get("SAREK_HIP_TEST_WALK_SEEDS", "12"))))
def test_random_walks_follow_the_reference_state_machine(hip, sarek, seed):
    E, V, T = sarek.Execute, sarek.Vector, sarek.Transfer
    rng = random.Random(seed)
    kernel = ("(kernel sarek_kern (params (param (var v 1 (vec f32))) (param (var n 2 i32))) (locals) (body "
              "(let (var tid 3 i32) (intr (Std) global_thread_id) (if (lt (var tid 3 i32) (var n 2 i32)) "
              "(assign (lelem v (var tid 3 i32)) (add (mul (read v (var tid 3 i32)) (f32 2.0)) (f32 1.0)))))) "
              "(native_fn true))")
    Model.auto_mode = True
    T.set_auto(True)
    parent_host = np.arange(64, dtype=np.float32)
    other_host = np.arange(40, dtype=np.float32) * np.float32(0.5)
    vectors = [V.of_array(parent_host.copy()), None, V.of_array(other_host.copy())]
    vectors[1] = vectors[0].sub_vector(8, 16)
    models = [Model(parent_host), None, Model(other_host)]
    models[1] = Model(parent_host[8:24])               # a view: writes go through to the parent's block
    steps = []

    def check(step):
        for k, (v, m) in enumerate(zip(vectors, models)):
            where = (seed, len(steps), step, k)
            assert v.location == m.location, (where, v.location, m.location, steps[-6:])
            assert np.array_equal(v.host, m.host), (where, steps[-6:])
            dev = device_contents(hip, v)
            assert (dev is None) == (m.device is None), (where, steps[-6:])
            if dev is not None:
                assert np.array_equal(dev, m.device), (where, steps[-6:])

    for _ in range(120):
        k = rng.randrange(len(vectors))
        v, m = vectors[k], models[k]
        op = rng.choice(["get", "set", "set", "fill", "to_device", "to_cpu", "to_cpu_force", "sync", "free", "launch",
                         "launch", "blit", "copy", "auto_sync", "auto_mode", "raw_write"])
        steps.append((op, k))
        if op == "get":
            i = rng.randrange(v.length)
            assert v.get(i) == m.get(i), (seed, steps[-6:])
        elif op == "set":
            i, x = rng.randrange(v.length), np.float32(rng.randint(-50, 50))
            v.set(i, x)
            m.set(i, x)
        elif op == "fill":
            x = np.float32(rng.randint(-9, 9))
            v.fill(x)
            m.fill(x)
        elif op == "to_device":
            T.to_device(v)
            m.to_device()
        elif op in ("to_cpu", "to_cpu_force"):
            T.to_cpu(v, force=op == "to_cpu_force")
            m.to_cpu(force=op == "to_cpu_force")
        elif op == "sync":
            T.sync(v)
            m.sync()
        elif op == "free":
            T.free_all_buffers(v)
            m.free_all_buffers()
        elif op == "launch":
            n = v.length
            assert E.run_vectors(kernel, [E.Vec(v), E.Int32(n)], (64, 1, 1), ((n + 63) // 64, 1, 1)) in ("jit", "map_f32")
            T.flush()
            m.launch()
        elif op == "blit":
            j = rng.randrange(len(vectors))
            src, src_m = vectors[j], models[j]
            length = rng.randint(0, min(8, src.length, v.length))
            so, do = rng.randint(0, src.length - length), rng.randint(0, v.length - length)
            V.blit(src, so, v, do, length)
            src_m.ensure_cpu_sync()
            for i in range(length):                    # element by element, ascending: ranges of one block may overlap
                m.host[do + i] = src_m.host[so + i]
                m.host_write()
        elif op == "copy":
            c = v.copy()
            m.ensure_cpu_sync()
            assert c.location == CPU and np.array_equal(c.host, m.host), (seed, steps[-6:])
        elif op == "auto_sync":
            flag = rng.random() < 0.6
            v.set_auto_sync(flag)
            m.auto_sync = flag
        elif op == "auto_mode":
            flag = rng.random() < 0.7
            T.set_auto(flag)
            Model.auto_mode = flag
        else:                                          # a write into the host block behind the vector's back
            i, x = rng.randrange(v.length), np.float32(rng.randint(100, 200))
            v.host[i] = x
            m.host[i] = x
        check(op)
    assert len({op for op, _ in steps}) >= 12
