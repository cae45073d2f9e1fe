"""Randomized differential test of the data-movement ops and the broadcast binary ops against numpy: shapes drawn from
extents on and off the vector grid and the 128-byte lines (1, 3, 8, 17, 63, 64, 65, 80, 1000, 1001, 1024 ...), every order
of permute, slices with ranges on and off the grid, broadcast patterns on either side, concats along every dim; a
third of the tensors large enough for the kernels that only large tensors take.  Bit equality (these ops move or add
values; numpy's result is the reference's)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

EXTENTS = [1, 2, 3, 4, 5, 7, 8, 12, 16, 17, 24, 31, 32, 33, 40, 63, 64, 65, 72, 80, 96, 100, 127, 128, 129, 200, 256, 300, 500, 512, 1000,
           1001, 1024, 1500, 2048]


@pytest.fixture(scope="module")
def dev():
    from ratchet_amd import Device

    d = Device(0)
    yield d
    d.close()


def _shape(rng, max_elems):
    while True:
        s = tuple(int(rng.choice(EXTENTS)) for _ in range(int(rng.integers(2, 5))))
        if int(np.prod(s)) <= max_elems:
            return s


def _same(got, want):
    bits = np.uint16 if want.dtype == np.float16 else np.uint32
    return got.shape == want.shape and np.array_equal(got.view(bits), want.view(bits))


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_shapes_against_numpy(dev, seed):
    rng = np.random.default_rng(seed)
    failures = []
    for it in range(240):
        kind = ("permute", "slice", "binary", "concat")[it % 4]
        dt = np.float16 if rng.integers(0, 2) else np.float32
        shape = _shape(rng, 6_000_000 if rng.integers(0, 3) == 0 else 200_000)
        x = rng.standard_normal(shape).astype(dt)
        if kind == "permute":
            perm = tuple(int(v) for v in rng.permutation(len(shape)))
            got, want, what = dev.permute(dev.upload(x), perm).to_numpy(), np.ascontiguousarray(x.transpose(perm)), (shape, perm)
        elif kind == "slice":
            ranges = []
            for d in shape:
                a = int(rng.integers(0, d))
                b = int(rng.integers(a + 1, d + 1))
                ranges.append((0, d) if rng.integers(0, 2) else (a, b))
            got = dev.slice(dev.upload(x), ranges).to_numpy()
            want, what = np.ascontiguousarray(x[tuple(slice(a, b) for a, b in ranges)]), (shape, ranges)
        elif kind == "binary":
            bshape = tuple(d if rng.integers(0, 2) else 1 for d in shape)
            k = int(rng.integers(0, len(shape)))
            if all(v == 1 for v in bshape[:k]):
                bshape = bshape[k:]                              # a lower-rank operand
            b = rng.standard_normal(bshape).astype(dt)
            op = ("add", "sub", "mul")[int(rng.integers(0, 3))]
            lhs, rhs = (b, x) if rng.integers(0, 2) else (x, b)
            got = dev.binary(op, dev.upload(lhs), dev.upload(rhs)).to_numpy()
            want = {"add": np.add, "sub": np.subtract, "mul": np.multiply}[op](lhs, rhs).astype(dt)
            what = (op, lhs.shape, rhs.shape)
        else:
            dim = int(rng.integers(0, len(shape)))
            other = list(shape)
            other[dim] = int(rng.choice([1, 3, 8, 17, 64]))
            y = rng.standard_normal(other).astype(dt)
            got = dev.concat([dev.upload(x), dev.upload(y)], dim).to_numpy()
            want, what = np.concatenate([x, y], axis=dim), (shape, tuple(other), dim)
        if not _same(got, want):
            failures.append((kind, np.dtype(dt).name, what))
    assert not failures, failures[:5]
