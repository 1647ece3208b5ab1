"""Seeded random sizes, alignments and distributions through the stream, layout and integer kernels, each case against
a reference computed on the device in float64 / int64 (what the mathematics fixes; the oracle-based tests of the same
kernels are tests/test_gpu_stream.py, test_gpu_layout.py, test_gpu_histogram.py):

  triad alone and fused with block sums, block maxima and the folded sum    the vector bit for bit ((double)b + (double)c * s
                                                                            rounded once); fused block sums and maxima the bits
                                                                            of the stand-alone block kernels
                                                                            total 1e-5
  block-256 sum, dot, maximum
  the fold                                     1e-5 of the sum of magnitudes
  maximum exact
  fold 1e-12
  copy, transpose                                                           exact, nothing stored outside the result
  five-point stencil, 3 x 3 box filter                                      bit for bit the double sums in the benches' order, one
                                                                            rounding; borders kept (stencil) or zero (filter)
  histogram (mod bins), radix histogram (shift, mask), radix scatter        exact counts on top of what the bins held
  output
                                                                            ordered by digit, the same keys per digit, counters
                                                                            at the ends of their ranges, nothing stored outside

Vectors start 0 to 64 elements into buffers that are NaN (inputs) or a guard value (outputs) everywhere else."""
import random

import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_seeded_random_cases(hip, torch_cuda, seed):
    torch = torch_cuda
    rng = random.Random(seed)
    failures = []

    def size():
        base = rng.choice([1, 3, 4, 255, 256, 257, 1023, 1024, 1025, 4095, 4096, 4097, 65535, 65536, 100003, 1 << 20,
                           (1 << 22) + 5, 3_000_001])
        return max(1, base + rng.choice([0, 0, 1, -1, 2, 3, rng.randint(0, 300)]))
    def view(n, dtype=torch.float32, fill=float("nan")):
        off = rng.choice([0, 1, 2, 3, 4, 7, 64])
        buf = torch.full((n + 200,), fill if dtype.is_floating_point else int(fill), device="cuda", dtype=dtype)
        return buf, buf[off:off + n], off
    def guard_ok(buf, off, n, fill):
        a, b = buf[:off], buf[off + n:]
        if isinstance(fill, float) and fill != fill:
            return bool(torch.isnan(a).all()) and bool(torch.isnan(b).all())
        return bool((a == fill).all()) and bool((b == fill).all())
    def block_ref(x, op, pad):
        n = x.numel()
        nb = (n + 255) // 256
        p = torch.full((nb * 256,), pad, device="cuda", dtype=torch.float64)
        p[:n] = x.double()
        p = p.view(nb, 256)
        return p.sum(1) if op == "sum" else p.max(1).values
    for it in range(150):
        def expect(ok, what):
            if not ok:
                failures.append((seed, it, kind, n, what))

        kind = rng.choice(["triad", "triad_bsum", "triad_bmax", "triad_sum", "bsum", "bmax", "dot", "fold", "copy",
                           "transpose", "hist", "rhist", "scatter", "stencil", "conv2d"])
        n = size()
        g = torch.Generator(device="cuda")
        g.manual_seed(it)
        if kind in ("triad", "triad_bsum", "triad_bmax", "triad_sum"):
            _, b, _ = view(n)
            _, c, _ = view(n)
            b.copy_(torch.randn(n, device="cuda", generator=g) * 3)
            c.copy_(torch.randn(n, device="cuda", generator=g))
            obuf, out, off = view(n, fill=7.0)
            s = rng.choice([3.0, -0.5, 1.0, 1e-3])
            s = torch.tensor(s, dtype=torch.float32).item()     # what the kernel receives
            want = (b.double() + c.double() * s).float()
            if kind == "triad":
                hip.triad(b, c, s, out=out)
            elif kind == "triad_bsum":
                _, sums = hip.triad_block256_sum(b, c, s, out=out)
                ref = hip.reduce_sum_block256(want)
                torch.cuda.synchronize()
                expect(torch.equal(sums.view(torch.int32), ref.view(torch.int32)), "bsum bits")
            elif kind == "triad_bmax":
                _, mx = hip.triad_block256_max(b, c, s, -1e6, out=out)
                ref = hip.reduce_max_block256(want, -1e6)
                torch.cuda.synchronize()
                expect(torch.equal(mx.view(torch.int32), ref.view(torch.int32)), "bmax bits")
            else:
                _, total = hip.triad_sum(b, c, s, out=out)
                torch.cuda.synchronize()
                w = want.double().sum().item()
                sc = want.double().abs().sum().item()
                expect(abs(total.item() - w) <= 1e-5 * max(sc, 1e-30), "total")
            torch.cuda.synchronize()
            expect(torch.equal(out.view(torch.int32), want.view(torch.int32)), "triad bits")
            expect(guard_ok(obuf, off, n, 7.0), "guard")
        elif kind in ("bsum", "bmax", "dot"):
            _, x, _ = view(n)
            x.copy_(torch.randn(n, device="cuda", generator=g) * 10)
            if kind == "dot":
                _, y, _ = view(n)
                y.copy_(torch.randn(n, device="cuda", generator=g))
                got = hip.dot_block256(x, y)
                ref = block_ref((x.double() * y.double()), "sum", 0.0)
                scale = block_ref((x.double() * y.double()).abs(), "sum", 0.0)
            elif kind == "bsum":
                got = hip.reduce_sum_block256(x)
                ref = block_ref(x, "sum", 0.0)
                scale = block_ref(x.abs(), "sum", 0.0)
            else:
                got = hip.reduce_max_block256(x, -1e6)
                ref = block_ref(x, "max", -1e6)
                scale = None
            torch.cuda.synchronize()
            if scale is None:
                expect(torch.equal(got.double(), ref), "max")
            else:
                expect(bool(((got.double() - ref).abs() <= 1e-5 * scale + 1e-30).all()), "block sums")
        elif kind == "fold":
            _, x, _ = view(n)
            x.copy_(torch.rand(n, device="cuda", generator=g) * 100)
            got = hip.fold_partials(x)
            torch.cuda.synchronize()
            w = x.double().sum().item()
            expect(abs(got.item() - w) <= 1e-12 * w, "fold")
        elif kind == "copy":
            _, x, _ = view(n)
            x.copy_(torch.randn(n, device="cuda", generator=g))
            obuf, out, off = view(n, fill=7.0)
            hip.copy(x, out=out)
            torch.cuda.synchronize()
            expect(torch.equal(out, x) and guard_ok(obuf, off, n, 7.0), "copy")
        elif kind == "transpose":
            h = rng.choice([1, 3, 16, 31, 64, 65, 127, 256, 300, 1000, 2049])
            w = rng.choice([1, 2, 16, 33, 64, 100, 128, 257, 512, 1001])
            _, x, _ = view(h * w)
            x.copy_(torch.randn(h * w, device="cuda", generator=g))
            obuf, out, off = view(h * w, fill=7.0)
            hip.transpose(x.view(h, w), out=out.view(w, h))
            torch.cuda.synchronize()
            expect(torch.equal(out.view(w, h), x.view(h, w).t()) and guard_ok(obuf, off, h * w, 7.0), "transpose")
        elif kind in ("stencil", "conv2d"):
            h = rng.choice([1, 2, 3, 4, 5, 17, 64, 65, 200, 777])
            w = rng.choice([1, 2, 3, 4, 5, 8, 63, 64, 65, 129, 256, 500, 1031])
            _, x, _ = view(h * w)
            x.copy_(torch.randn(h * w, device="cuda", generator=g) * 10.0 ** rng.randint(-3, 3))
            obuf, out, off = view(h * w, fill=7.0)
            g2, d = x.view(h, w), x.view(h, w).double()
            want = torch.full((h, w), 7.0 if kind == "stencil" else 0.0, device="cuda")
            if h > 2 and w > 2:
                if kind == "stencil":          # up + down + left + right + center, in double, / 5.0, one rounding
                    inner = (d[:-2, 1:-1] + d[2:, 1:-1] + d[1:-1, :-2] + d[1:-1, 2:] + d[1:-1, 1:-1]) / 5.0
                else:                          # the nine cells row by row, in double, / 9.0, one rounding
                    inner = d[:-2, :-2] + d[:-2, 1:-1] + d[:-2, 2:]
                    inner = inner + d[1:-1, :-2] + d[1:-1, 1:-1] + d[1:-1, 2:]
                    inner = (inner + d[2:, :-2] + d[2:, 1:-1] + d[2:, 2:]) / 9.0
                want[1:-1, 1:-1] = inner.float()
            (hip.stencil_2d if kind == "stencil" else hip.conv2d)(g2, out=out.view(h, w))
            torch.cuda.synchronize()
            n = (h, w)
            expect(torch.equal(out.view(h, w).view(torch.int32), want.view(torch.int32)), "grid bits")
            expect(guard_ok(obuf, off, h * w, 7.0), "guard")
        elif kind in ("hist", "rhist"):
            bins = rng.choice([1, 2, 7, 16, 100, 255, 256])
            _, keys, _ = view(n, torch.int32, 0)
            dist = rng.choice(["uniform", "one", "few", "neg"])
            if dist == "uniform": keys.copy_(torch.randint(0, 1 << 30, (n,), device="cuda", generator=g, dtype=torch.int32))
            elif dist == "one": keys.fill_(rng.randint(0, 1 << 20))
            elif dist == "few": keys.copy_(torch.randint(0, 3, (n,), device="cuda", generator=g, dtype=torch.int32) * 77 + 5)
            else: keys.copy_(torch.randint(-(1 << 30), 1 << 30, (n,), device="cuda", generator=g, dtype=torch.int32))
            hist = torch.randint(0, 5, (256,), device="cuda", dtype=torch.int32)
            before = hist.clone()
            if kind == "hist":
                if dist == "neg": keys.abs_()
                hip.histogram(keys, hist, bins)
                torch.cuda.synchronize()
                ref = torch.bincount((keys.long() % bins), minlength=256).int() + before
            else:
                shift = rng.choice([0, 8, 16, 24])
                mask = rng.choice([255, 15, 127])
                hip.radix_histogram(keys, hist, shift, mask)
                torch.cuda.synchronize()
                ref = torch.bincount(((keys.long() & 0xFFFFFFFF) >> shift) & mask, minlength=256).int() + before
            expect(torch.equal(hist, ref), "hist")
        else:
            n = min(n, 1 << 22)
            shift = rng.choice([0, 8, 16, 24])
            _, keys, _ = view(n, torch.int32, 0)
            if rng.random() < 0.7:
                keys.copy_(torch.randint(0, 1 << 30, (n,), device="cuda", generator=g, dtype=torch.int32))
            else:                                        # four digits only
                keys.copy_(torch.randint(0, 4, (n,), device="cuda", generator=g, dtype=torch.int32) << shift)
            digit = ((keys.long() >> shift) & 255)
            counts = torch.bincount(digit, minlength=256)
            starts = (torch.cumsum(counts, 0) - counts).int()
            counters = starts.clone()
            obuf, out, off = view(n, torch.int32, -5)
            hip.radix_scatter(keys, out, counters, shift)
            torch.cuda.synchronize()
            ok = torch.equal(counters.long(), starts.long() + counts) and guard_ok(obuf, off, n, -5)
            od = ((out.long() >> shift) & 255)
            ok = ok and torch.equal(od, torch.sort(digit).values)          # ordered by digit
            ok = ok and torch.equal(torch.sort(out).values, torch.sort(keys).values)   # same multiset overall
            # same multiset per digit: sort by (digit, key)
            ok = ok and torch.equal(torch.sort(od * (1 << 32) + (out.long() & 0xFFFFFFFF)).values,
                                    torch.sort(digit * (1 << 32) + (keys.long() & 0xFFFFFFFF)).values)
            expect(ok, "scatter")
    assert failures == []
