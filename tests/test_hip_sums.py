"""GPU parity of the sums against the oracle beyond the golden cases: the parallel
evaluation of sum1d on data that crosses binades, changes sign, ties, hovers at binade
edges, holds infinities / NaNs / zeros, on odd lengths and unaligned pointers; and the
row / column / channel sums on shapes around the tile sizes."""
import numpy as np
import pytest
import torch

import gen
from oracle import api as oracle

pytestmark = pytest.mark.gpu


def _rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def _cases():
    r = _rng(11)
    n = 300_000
    yield "uniform_pm1", gen.uniform_pm1(1, 1_000_003).numpy()
    yield "scaled_normal", gen.scaled_normal(2, 777_777).numpy()
    yield "positive_drift", (r.random(n) * 3).astype(np.float32)
    yield "negative_drift", (-r.random(n) * 3).astype(np.float32)
    yield "hover_edge", np.concatenate([[1024.0], np.where(r.random(n) < 0.5, 1.0, -1.0) + r.standard_normal(n) * 1e-3]).astype(np.float32)
    yield "ties", np.concatenate([[2.0**24], np.ones(100_000), [-2.0**23], np.full(100_000, 0.5)]).astype(np.float32)
    yield "tiny_after_big", np.concatenate([[1e8], r.random(n) * 1e-3, [-1e8], r.random(n)]).astype(np.float32)
    yield "zeros", np.zeros(200_000, dtype=np.float32)
    yield "zeros_then_values", np.concatenate([np.zeros(70_000), -np.zeros(5_000), r.standard_normal(100_000)]).astype(np.float32)
    yield "inf_nan", np.concatenate([r.standard_normal(90_000), [np.inf], r.standard_normal(50_000), [-np.inf], r.standard_normal(50_000)]).astype(np.float32)
    yield "subnormal_state", (r.integers(-2**20, 2**20, n).astype(np.float64) * 2.0**-149).astype(np.float32)
    yield "cancel_to_zero", np.tile(np.array([3.25, -3.25, 1e-3, -1e-3], dtype=np.float32), 60_000)
    # the running sum stops growing at 2^24 (every element below half a quantum) two thirds
    # of the way through, and at 2^22 for the smaller elements that follow a large start
    yield "stagnation", (0.25 + 0.75 * r.random(1 << 25)).astype(np.float32)
    yield "stagnation_small", np.concatenate([[2.0**22], r.random(2_000_000) * 0.25, -r.random(500_000) * 0.3]).astype(np.float32)
    yield "just_long_enough", gen.uniform_pm1(3, 12288).numpy()
    yield "just_too_short", gen.uniform_pm1(4, 12287).numpy()


@pytest.mark.parametrize("name,x", list(_cases()), ids=[n for n, _ in _cases()])
def test_sum1d_parallel_path(name, x):
    from repdl_amd import ops

    t = torch.from_numpy(np.ascontiguousarray(x))
    for avg in (False, True):
        got = ops.sum1d(t.cuda(), avg).cpu()
        want = oracle.sum1d(t, avg)
        assert got.shape == want.shape
        assert got.view(torch.int32).item() == want.view(torch.int32).item() or (torch.isnan(got) and torch.isnan(want)), (name, avg)


@pytest.mark.parametrize("n", [12288, 12289, 16384, 20_000, 32767, 32768, 36865, 65536, 65537, 100_001, 131_072, 200_000, 262_143])
def test_sum1d_one_short_chain(n):
    """One chain shorter than 2^18 elements takes two launches (the map pass predicts the state at its own
    block's start, the walk joins the one super-block's tuple): lengths at and off block boundaries, data that
    drifts, changes sign and hovers near zero, pointers on and off 16-byte boundaries, sum and mean."""
    from repdl_amd import ops

    r = _rng(n)
    kinds = {"zero_mean": r.random(n + 1) * 2 - 1, "drift": r.random(n + 1) * 10 + 2, "normal": r.standard_normal(n + 1),
             "negative_drift": -r.random(n + 1)}
    for name, v in kinds.items():
        h = torch.from_numpy(v.astype(np.float32))
        d = h.cuda()
        for off in (0, 1):
            for avg in (False, True):
                got, want = ops.sum1d(d[off:], avg).cpu(), oracle.sum1d(h[off:], avg)
                assert got.view(torch.int32).item() == want.view(torch.int32).item(), (name, off, avg)


def test_sum1d_unaligned_and_plain_entry():
    """Unaligned input pointer, and the C entry point without a workspace (which takes
    its scratch from the stream-ordered allocator)."""
    import ctypes

    from repdl_amd import _lib, ops

    buf = gen.uniform_pm1(5, 400_001).cuda()
    x = buf[1:]
    assert x.data_ptr() % 16 != 0
    want = oracle.sum1d(x.cpu())
    assert torch.equal(ops.sum1d(x).cpu(), want)
    out = torch.empty((), dtype=torch.float32, device="cuda")
    _lib.call("repdl_hip_sum1d", ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(out.data_ptr()), x.numel(), 0,
              ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), want)
    small = ctypes.c_size_t(16)
    rc = _lib.lib().repdl_hip_sum1d_ws(ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(out.data_ptr()), x.numel(), 0,
                                       ctypes.c_void_p(buf.data_ptr()), small, None)
    assert rc == -3  # workspace too small


@pytest.mark.parametrize("shape", [(1, 5000), (3, 8193), (17, 511), (100, 100), (6200, 300), (13000, 65), (50000, 33)])
def test_row_and_column_sums(shape):
    from repdl_amd import ops

    M, N = shape
    x = gen.scaled_normal(M + N, M, N)
    for avg in (False, True):
        assert torch.equal(ops.sum2d_dim1(x.cuda(), False, avg).cpu(), oracle.sum2d_dim1(x, False, avg))
        assert torch.equal(ops.sum2d_dim0(x.cuda(), True, avg).cpu(), oracle.sum2d_dim0(x, True, avg))
    xu = gen.scaled_normal(7, M * N + 1).cuda()[1:].view(M, N)  # unaligned rows
    assert torch.equal(ops.sum2d_dim1(xu).cpu(), oracle.sum2d_dim1(xu.cpu()))


@pytest.mark.parametrize("shape", [(2, 3, 5, 7), (4, 64, 14, 14), (3, 130, 8, 8), (1, 7000, 3, 3),
                                   # several whole segments per tile row: full and ragged last tiles, widths that are
                                   # not multiples of 4, more chains per workgroup
                                   (64, 16, 14, 14), (5, 8, 28, 28), (7, 4, 33, 31), (3, 6200, 4, 4), (23, 5, 2, 2),
                                   (4, 2, 32, 32), (3, 2, 33, 32)])
def test_channel_sums(shape):
    from repdl_amd import ops

    x = gen.scaled_normal(sum(shape), *shape)
    assert torch.equal(ops.sum4d_dim023(x.cuda()).cpu(), oracle.sum4d_dim023(x))
    assert torch.equal(ops.sum(x.cuda(), dim=(0, 2, 3), keepdim=True, average=True).cpu(), oracle.sum4d_dim023(x, True, True))


@pytest.mark.parametrize("shape", [(9, 5, 14, 14), (3, 7, 28, 28), (6, 3, 5, 7)])
def test_channel_sums_unaligned_pointer(shape):
    """An input that starts 4 bytes off a 16-byte boundary: the scalar loads of the loader, with
    several segments per tile row."""
    from repdl_amd import ops

    n = shape[0] * shape[1] * shape[2] * shape[3]
    flat = gen.scaled_normal(77, n + 1)
    x = flat[1:].view(*shape)
    xd = flat.cuda()[1:].view(*shape)
    assert xd.data_ptr() % 16 != 0
    assert torch.equal(ops.sum4d_dim023(xd).cpu(), oracle.sum4d_dim023(x.contiguous()))


def _long_rows():
    """Few, long chains: row sums and channel sums that take the parallel evaluation (chains of at
    least 49152 elements, at most 512 of them, or at most 64 of at least 24576), with the data that attacks it."""
    r = _rng(12)
    L = 70_000
    rows = [
        gen.uniform_pm1(7, L).numpy(),
        (r.random(L) * 3).astype(np.float32),
        np.concatenate([[1024.0], np.where(r.random(L - 1) < 0.5, 1.0, -1.0) + r.standard_normal(L - 1) * 1e-3]).astype(np.float32),
        np.concatenate([[2.0**24], np.ones(L // 2 - 1), [-2.0**23], np.full(L - L // 2 - 1, 0.5)]).astype(np.float32),
        np.zeros(L, dtype=np.float32),
        np.concatenate([r.standard_normal(L // 2), [np.inf], r.standard_normal(L - L // 2 - 1)]).astype(np.float32),
        (r.integers(-2**20, 2**20, L).astype(np.float64) * 2.0**-149).astype(np.float32),
        np.tile(np.array([3.25, -3.25, 1e-3, -1e-3], dtype=np.float32), L // 4),
    ]
    return np.stack(rows)


def test_row_sums_few_long_rows():
    from repdl_amd import ops

    m = torch.from_numpy(_long_rows())  # 8 x 70000 (70000 % 16 == 0)
    got, want = ops.sum2d_dim1(m.cuda()).cpu(), oracle.sum2d_dim1(m)
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(got), nan) and torch.equal(got[~nan].view(torch.int32), want[~nan].view(torch.int32))
    m2 = gen.scaled_normal(90, 5, 65537)  # a row length that is no multiple of 4: scalar loads
    assert torch.equal(ops.sum2d_dim1(m2.cuda()).cpu(), oracle.sum2d_dim1(m2))
    for n in (24575, 24576, 24592, 49151, 49152, 49168):  # either side of the lengths at which rows change kernels
        for rows in (3, 65):                                 # (up to 64 chains from 24576 elements, up to 512 from 49152)
            m4 = gen.uniform_pm1(92 + n, rows, n)
            assert torch.equal(ops.sum2d_dim1(m4.cuda()).cpu(), oracle.sum2d_dim1(m4)), (rows, n)
    m3 = gen.uniform_pm1(91, 300, 66000)
    assert torch.equal(ops.sum2d_dim1(m3.cuda(), average=True).cpu(), oracle.sum2d_dim1(m3, average=True))


@pytest.mark.parametrize("shape", [(8, 5, 96, 96), (3, 4, 160, 144), (70, 3, 32, 32), (9, 2, 90, 90), (2, 64, 224, 224),
                                   (64, 8, 28, 28), (48, 3, 32, 32), (47, 3, 32, 32)])
def test_channel_sums_few_long_chains(shape):
    """Channel sums whose chains (N*H*W elements) are long and few: a segment per image; (9, 2, 90, 90)
    has segments that are no multiple of 16 and stays with the row-chain kernel."""
    from repdl_amd import ops

    x = gen.uniform_pm1(sum(shape), *shape) if shape[0] != 3 else gen.scaled_normal(5, *shape)
    assert torch.equal(ops.sum4d_dim023(x.cuda()).cpu(), oracle.sum4d_dim023(x))
    xr = x.clamp(min=0)
    assert torch.equal(ops.sum4d_dim023(xr.cuda(), average=True).cpu(), oracle.sum4d_dim023(xr, average=True))
    n = x.numel()
    flat = torch.cat([torch.zeros(1), x.view(-1)]).cuda()
    xd = flat[1:].view(*shape)  # 4 bytes off a 16-byte boundary
    assert xd.data_ptr() % 16 != 0
    assert torch.equal(ops.sum4d_dim023(xd).cpu(), oracle.sum4d_dim023(x))


def test_full_size_benchmark_inputs():
    """The two inputs of the sum configuration at their full sizes: 2^28 uniform multiples of
    2^-23 in [-1, 1) through sum1d, and row sums of a 16384 x 16384 matrix of N(0,1) values
    scaled by 2^U[-20,20]; every output bit against the oracle."""
    from repdl_amd import ops

    x = gen.uniform_pm1(2028, 1 << 28)
    for avg in (False, True):
        got = ops.sum1d(x.cuda(), avg).cpu()
        assert got.view(torch.int32).item() == oracle.sum1d(x, avg).view(torch.int32).item(), avg
    # a drifting input of the same length: the running sum stops growing at 2^24
    y = x.abs_()
    assert ops.sum1d(y.cuda()).cpu().view(torch.int32).item() == oracle.sum1d(y).view(torch.int32).item()
    del x, y
    m = gen.scaled_normal(2029, 16384, 16384)
    got = ops.sum2d_dim1(m.cuda()).cpu()
    assert torch.equal(got.view(torch.int32), oracle.sum2d_dim1(m).view(torch.int32))
    assert torch.equal(ops.sum2d_dim0(m.cuda()).cpu().view(torch.int32), oracle.sum2d_dim0(m).view(torch.int32))


def _long_cases():
    """Inputs long enough for the speculative rounds of the single-chain evaluation (2^22 elements
    and more), built to make the rounds miss: sums that cross zero and many binades, that fall from
    a large magnitude to a small one, that stop growing at a power of two, that pass through
    infinities and NaNs, all-zero stretches, and lengths that fill the last block, node or
    super-block only partly."""
    r = _rng(31)
    n = (1 << 22) + 12345
    yield "uniform_pm1_ragged", gen.uniform_pm1(41, n).numpy()
    yield "exactly_2^22", gen.uniform_pm1(42, 1 << 22).numpy()
    yield "one_node_short", gen.uniform_pm1(43, (1 << 23) - 16384 + 7).numpy()
    yield "normal_full_mantissa", r.standard_normal(n).astype(np.float32)
    down = np.concatenate([[3.0e6], -np.abs(r.standard_normal(3_000_000)).astype(np.float32) * 1.2, r.standard_normal(1_500_000)])
    yield "descent", down.astype(np.float32)
    yield "stagnation_at_2^24", (0.25 + 0.75 * r.random(1 << 25)).astype(np.float32)
    z = r.standard_normal(n).astype(np.float32)
    z[1_000_000:1_300_000] = 0.0
    z[2_000_000:2_000_064] = -0.0
    yield "zero_stretches", z
    w = r.standard_normal(n).astype(np.float32)
    w[3_000_001] = np.inf
    yield "inf_late", w
    v = r.standard_normal(n).astype(np.float32)
    v[2_500_000], v[2_500_777] = np.inf, -np.inf
    yield "nan_midway", v
    yield "scaled_normal", gen.scaled_normal(44, n).numpy()
    yield "tiny_values", (r.standard_normal(n) * 2.0**-140).astype(np.float32)
    yield "huge_values", (r.standard_normal(n) * 2.0**100).astype(np.float32)


@pytest.mark.parametrize("name,x", list(_long_cases()), ids=[n for n, _ in _long_cases()])
def test_sum1d_speculative_rounds(name, x):
    from repdl_amd import ops

    t = torch.from_numpy(np.ascontiguousarray(x))
    got = ops.sum1d(t.cuda(), name == "descent").cpu()
    want = oracle.sum1d(t, name == "descent")
    assert got.view(torch.int32).item() == want.view(torch.int32).item() or (torch.isnan(got) and torch.isnan(want)), name


def test_rounds_on_chains_in_rows():
    """Row sums and channel sums whose chains are long enough (2^19 elements and more) for the speculative
    rounds: every row a different kind of trouble -- zero crossings, a fall through many binades, stagnation
    at a power of two, zero stretches, an infinity, NaNs, tiny and huge magnitudes -- and ragged lengths."""
    from repdl_amd import ops

    r = _rng(77)
    n = (1 << 19) + 4321
    rows = []
    rows.append(r.standard_normal(n))
    rows.append(r.random(n) * 2 - 1)
    d = r.standard_normal(n)
    d[0] = 3.0e5
    d[1:200_000] = -np.abs(d[1:200_000]) * 1.5
    rows.append(d)
    rows.append(0.25 + 0.75 * r.random(n))                 # keeps growing
    rows.append((0.25 + 0.75 * r.random(n)) * 2.0**7)      # stops growing at 2^24 * 2^7 / ... within the row
    z = r.standard_normal(n)
    z[50_000:120_000] = 0.0
    z[130_000:130_064] = -0.0
    rows.append(z)
    w = r.standard_normal(n)
    w[200_001] = np.inf
    rows.append(w)
    v = r.standard_normal(n)
    v[100_000], v[100_777] = np.inf, -np.inf
    rows.append(v)
    rows.append(r.standard_normal(n) * 2.0**-140)
    rows.append(r.standard_normal(n) * 2.0**100)
    rows.append(gen.scaled_normal(78, n).numpy())
    rows.append(np.zeros(n))
    m = torch.from_numpy(np.stack(rows).astype(np.float32))
    for avg in (False, True):
        got = ops.sum2d_dim1(m.cuda(), False, avg).cpu()
        want = oracle.sum2d_dim1(m, False, avg)
        same = (got.view(torch.int32) == want.view(torch.int32)) | (torch.isnan(got) & torch.isnan(want))
        assert bool(same.all()), (avg, torch.nonzero(~same).flatten().tolist())
    # two rows long enough for more than 16 super-blocks each (the round's kernels stay separate there)
    m2 = torch.from_numpy(np.stack([r.standard_normal((1 << 23) + 77), r.random((1 << 23) + 77) - 0.5]).astype(np.float32))
    got = ops.sum2d_dim1(m2.cuda()).cpu()
    assert torch.equal(got.view(torch.int32), oracle.sum2d_dim1(m2).view(torch.int32))
    # seventy rows of 33 nodes each: 2310 nodes, more than one pass of the round's walkers
    m3 = torch.from_numpy(r.standard_normal((70, (1 << 19) + 5)).astype(np.float32))
    m3[::7] += 0.25
    m3[3] *= 2.0**40
    got = ops.sum2d_dim1(m3.cuda()).cpu()
    assert torch.equal(got.view(torch.int32), oracle.sum2d_dim1(m3).view(torch.int32))
    del m3
    # channel sums: 8 channels of 48 images of 112x112 (602112 elements per chain), zero-mean and shifted channels
    x = torch.from_numpy(r.standard_normal((48, 8, 112, 112)).astype(np.float32))
    x[:, 3] += 0.5
    x[:, 5] = x[:, 5].abs()
    x[:, 7] *= 2.0**-130
    x[7, 2, 3, 3] = float("inf")
    got = ops.sum4d_dim023(x.cuda()).cpu()
    want = oracle.sum4d_dim023(x)
    same = (got.view(torch.int32) == want.view(torch.int32)) | (torch.isnan(got) & torch.isnan(want))
    assert bool(same.all()), torch.nonzero(~same).flatten().tolist()


def test_sum1d_long_unaligned_and_workspace():
    """A long chain from a pointer 4 bytes off a 16-byte boundary, and the same through the entry point
    that takes the caller's scratch memory (deliberately filled with junk first)."""
    import ctypes

    from repdl_amd import _lib, ops

    n = (1 << 22) + 999
    buf = gen.uniform_pm1(51, n + 1).cuda()
    x = buf[1:]
    assert x.data_ptr() % 16 != 0
    want = oracle.sum1d(x.cpu())
    assert torch.equal(ops.sum1d(x).cpu(), want)
    nb = _lib.lib().repdl_hip_sum1d_workspace_bytes(n)
    ws = torch.randint(0, 255, (nb,), dtype=torch.uint8, device="cuda")
    out = torch.empty((), dtype=torch.float32, device="cuda")
    for _ in range(2):  # the second call finds the first call's leftovers
        _lib.call("repdl_hip_sum1d_ws", ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(out.data_ptr()), n, 0,
                  ctypes.c_void_p(ws.data_ptr()), ctypes.c_size_t(nb), None)
        torch.cuda.synchronize()
        assert torch.equal(out.cpu(), want)
