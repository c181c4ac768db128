"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle.

Tolerances (max relative error per tensor, tests/parity.py): 1e-5 for fp32,
2e-3 for fp16 storage with fp32 accumulation.  Where the fp32 reference is itself
further than that from the float64 evaluation of the same algorithm, a result at
least as close to float64 as the reference is also accepted (parity.check).
"""
import numpy as np
import pytest
import torch

from oracle import cpu_oracle as orc
from tests.parity import TOL_F16, TOL_F32, check, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def L():
    from lbann_amd import layers
    layers.capi.lib()  # fail loudly if the library is missing
    assert torch.cuda.is_available()
    return layers


def f64(a):
    return np.asfortranarray(np.asarray(a, dtype=np.float64))


def f32(a):
    return np.asfortranarray(np.asarray(a, dtype=np.float32))


def rand(rng, h, w, mean=0.0, std=1.0):
    return np.asfortranarray((rng.standard_normal((w, h)) * std + mean).astype(np.float32).T)


# ===================================================================== softmax family
SM_SHAPES = [
    # (h, w, ld_pad)   register path: one wave / 256 / 1024 threads per row, all vector counts
    (64, 5, 0), (256, 9, 0), (1000, 7, 0), (1024, 33, 0), (2048, 6, 0), (4096, 10, 0),
    (8192, 4, 0), (12288, 3, 0), (32768, 3, 0), (20000, 2, 0),
    (512, 7, 64),          # ld > height (a view into a taller matrix), still 16-byte aligned
    (7, 19, 0), (31, 5, 0), (1001, 4, 0), (130, 3, 3),   # unaligned / odd heights: scalar split kernels
    (32772, 2, 0), (70000, 3, 0), (262144, 2, 0),        # longer than the register path: split kernels
    (262148, 48, 0), (100000, 130, 0),                   # long rows, large footprint: register-resident clusters
    (1, 6, 0),
    # rows that are only 4-byte aligned: one float per access in registers up to 32768 entries;
    # beyond, the cluster kernels with one float per access when the tensor is large, else
    # 16-byte accesses with scalar edges in the split kernels
    (197, 70, 0), (8191, 9, 0), (8193, 3, 0), (30522, 5, 0), (50257, 6, 0), (10, 300, 0), (4099, 7, 1),
    (16383, 5, 0), (16385, 4, 0), (32767, 3, 0), (32769, 3, 0), (50257, 270, 0), (131071, 101, 0), (131075, 101, 0),
    (40001, 700, 1),       # more rows than resident clusters
    # many short rows: teams of 16 lanes, four rows per wave (vector and single-float access)
    (16, 5000, 0), (64, 4100, 0), (128, 4096, 0), (200, 4500, 0), (256, 4097, 0), (10, 5000, 0), (49, 6000, 0),
    (63, 4096, 1), (12, 4095, 0),
]


def _sm_oracle(kind):
    return {"softmax": (orc.softmax_fwd, orc.softmax_bwd),
            "log_softmax": (orc.log_softmax_fwd, orc.log_softmax_bwd)}[kind]


@pytest.mark.parametrize("kind", ["softmax", "log_softmax"])
@pytest.mark.parametrize("h,w,pad", SM_SHAPES)
def test_softmax_family(L, kind, h, w, pad):
    rng = np.random.default_rng(h * 1000 + w)
    x, dy = rand(rng, h, w, 0, 2), rand(rng, h, w)
    if h > 8:
        x[rng.integers(0, h, size=max(1, h // 100)), :] = 30.0
    fwd, bwd = _sm_oracle(kind)
    layer = L.softmax_layer() if kind == "softmax" else L.log_softmax_layer()
    ld = h + pad
    y = layer.forward(L.DeviceMatrix.from_numpy(x, ldim=ld)).to_numpy()
    y_ref, y_ex = fwd(x), fwd(f64(x))
    check(f"{kind} y {h}x{w}", y, y_ref, y_ex)
    # backward consumes the layer's own output, as in the framework
    dx = layer.backward(L.DeviceMatrix.from_numpy(dy, ldim=ld)).to_numpy()
    check(f"{kind} dx {h}x{w}", dx, bwd(f32(y), dy), bwd(f64(y), f64(dy)))


@pytest.mark.parametrize("kind", ["softmax", "log_softmax"])
@pytest.mark.parametrize("h,w,pad,in_place", [
    (1000, 37, 0, False), (4096, 64, 0, False), (32768, 48, 0, True), (65536, 9, 0, False),   # 16-byte vectors
    (197, 50, 0, False), (1001, 33, 3, False), (16385, 6, 0, True),                          # single halves
    (64, 5000, 0, False), (24, 4099, 0, False),                                             # short rows, 16-lane teams
    (70000, 3, 0, False), (40001, 2, 0, True), (131072, 2, 0, False),                        # beyond the register kernels
    (32768, 300, 0, True), (20480, 513, 0, False), (24584, 260, 8, False),    # more rows than compute units: walked
    (128256, 40, 0, True), (65544, 5, 8, False), (65540, 3, 0, False),        # long rows: two packed passes,
    (50257, 9, 0, True), (40001, 5, 16, False), (33001, 7, 0, False), (32770, 4, 3, False),  # cut at 16-byte boundaries per row
    (1003, 33, 0, True), (4099, 9, 1, True), (259, 5000, 0, True),   # unaligned vectors, in place
])
def test_softmax_family_f16_storage(L, kind, h, w, pad, in_place):
    """fp16 storage, fp32 arithmetic (softmax.cpp:236-243 instantiates the layers for half):
    both sides see the fp16-rounded inputs; the oracle is the fp32 restatement on them."""
    rng = np.random.default_rng(3 * h + w)
    x16 = rand(rng, h, w, 0, 2).astype(np.float16)
    dy16 = rand(rng, h, w).astype(np.float16)
    x, dy = f32(x16), f32(dy16)
    layer = L.softmax_layer() if kind == "softmax" else L.log_softmax_layer()
    fwd, bwd = _sm_oracle(kind)
    ld = h + pad
    xm = L.DeviceMatrix.from_numpy(x16, dtype=torch.float16, ldim=ld)
    ym = layer.forward(xm, in_place=in_place)
    assert ym.dtype == torch.float16 and (ym is xm) == in_place
    y = ym.to_numpy()
    check(f"{kind} f16 y {h}x{w}", y, fwd(x), fwd(f64(x)), tol=TOL_F16)
    gm = L.DeviceMatrix.from_numpy(dy16, dtype=torch.float16, ldim=ld)
    dx = layer.backward(gm, in_place=in_place).to_numpy()
    # backward consumes the layer's own (fp16) output, as in the framework
    check(f"{kind} f16 dx {h}x{w}", dx, bwd(f32(y), dy), bwd(f64(y), f64(dy)), tol=TOL_F16)
    if kind == "softmax":
        assert np.abs(y.astype(np.float64).sum(axis=0) - 1).max() < 2e-3 * np.sqrt(h)


@pytest.mark.parametrize("kind", ["softmax", "log_softmax"])
@pytest.mark.parametrize("h,w,pad", [
    (9, 50, 0), (15, 5000, 0), (17, 4100, 1), (63, 40, 0), (65, 4200, 0), (129, 33, 0), (255, 5000, 0), (257, 700, 0),
    (511, 64, 3), (513, 4100, 0), (1023, 9, 0), (1025, 70, 0), (2047, 12, 0), (2049, 300, 0), (3001, 17, 0),
    (4095, 5, 0), (4097, 40, 0), (8191, 6, 0), (16385, 7, 0), (24001, 3, 0), (32767, 4, 0), (50001, 3, 0),
    # whole eights of entries behind odd leading dimensions: no partial vector, still unaligned
    (1024, 9, 1), (64, 5000, 3), (2048, 33, 5), (16, 4100, 1)])
def test_softmax_family_f16_unaligned_rows(L, kind, h, w, pad):
    """fp16 rows that are not whole aligned vectors, in 16-byte accesses at 2-byte alignment: the row's
    last h % 8 entries come from a vector that overlaps its neighbour."""
    rng = np.random.default_rng(7 * h + w + pad)
    x16 = rand(rng, h, w, 0, 2).astype(np.float16)
    x16[h - 1, ::3] = 9.0   # the maximum in the partial vector, or in its neighbour
    x16[max(h - 9, 0), 1::3] = 9.0
    dy16 = rand(rng, h, w).astype(np.float16)
    x, dy = f32(x16), f32(dy16)
    layer = L.softmax_layer() if kind == "softmax" else L.log_softmax_layer()
    fwd, bwd = _sm_oracle(kind)
    y = layer.forward(L.DeviceMatrix.from_numpy(x16, dtype=torch.float16, ldim=h + pad)).to_numpy()
    check(f"{kind} f16 y {h}x{w}", y, fwd(x), fwd(f64(x)), tol=TOL_F16)
    dx = layer.backward(L.DeviceMatrix.from_numpy(dy16, dtype=torch.float16, ldim=h + pad)).to_numpy()
    check(f"{kind} f16 dx {h}x{w}", dx, bwd(f32(y), dy), bwd(f64(y), f64(dy)), tol=TOL_F16)
    if kind == "softmax":
        assert np.abs(y.astype(np.float64).sum(axis=0) - 1).max() < 2e-3 * np.sqrt(h)


@pytest.mark.parametrize("h", [13, 259, 1027])
def test_softmax_f16_special_values_on_unaligned_rows(L, h):
    """-inf, a dominant entry and NaN in the partial vector at the end of an odd row and in its neighbour."""
    x = np.zeros((h, 5), dtype=np.float16)
    x[:, 0] = 3.0
    x[h - 1, 1] = 60000.0
    x[:, 2] = -np.inf
    x[h - 2, 2] = 1.0
    x[h - 1, 3] = np.nan
    x[h - 9, 4] = np.nan
    layer = L.softmax_layer()
    y = layer.forward(L.DeviceMatrix.from_numpy(x, dtype=torch.float16)).to_numpy()
    ref = orc.softmax_fwd(f32(x))
    assert np.allclose(y[:, 0], 1.0 / h, rtol=2e-3)
    assert y[h - 1, 1] == 1.0 and y[:, 1].sum() == 1.0
    assert y[h - 2, 2] == 1.0 and y[:, 2].sum() == 1.0
    assert (ref[:, 3:] == 0).all() and (y[:, 3:] == 0).all()
    ls = L.log_softmax_layer()
    yl = ls.forward(L.DeviceMatrix.from_numpy(x[:, :3], dtype=torch.float16)).to_numpy()
    refl = orc.log_softmax_fwd(f32(x[:, :3]))
    assert np.array_equal(np.isneginf(yl), np.isneginf(refl))
    fin = np.isfinite(refl)
    assert np.allclose(yl[fin], refl[fin], rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("kind", ["softmax", "log_softmax"])
@pytest.mark.parametrize("h,w,pad", [(2049, 70, 0), (2050, 9, 0), (3001, 17, 0), (3071, 300, 0), (4095, 5, 0),
                                     (4096, 9, 1), (3072, 12, 3), (2052, 7, 2)])
def test_softmax_family_f32_unaligned_rows(L, kind, h, w, pad):
    """fp32 rows of 2049 to 4096 entries off the 16-byte grid, in 16-byte accesses at 4-byte alignment."""
    rng = np.random.default_rng(5 * h + w + pad)
    x, dy = rand(rng, h, w, 0, 2), rand(rng, h, w)
    x[h - 1, ::3] = 30.0
    x[h - 5, 1::3] = 30.0
    fwd, bwd = _sm_oracle(kind)
    layer = L.softmax_layer() if kind == "softmax" else L.log_softmax_layer()
    y = layer.forward(L.DeviceMatrix.from_numpy(x, ldim=h + pad)).to_numpy()
    check(f"{kind} y {h}x{w}", y, fwd(x), fwd(f64(x)))
    dx = layer.backward(L.DeviceMatrix.from_numpy(dy, ldim=h + pad)).to_numpy()
    check(f"{kind} dx {h}x{w}", dx, bwd(f32(y), dy), bwd(f64(y), f64(dy)))


def test_softmax_f16_special_values(L):
    """A column of equal values, one with a dominant entry, one with -inf entries, one NaN."""
    h = 256
    x = np.zeros((h, 4), dtype=np.float16)
    x[:, 0] = 3.0
    x[7, 1] = 60000.0
    x[:, 2] = -np.inf
    x[5, 2] = 1.0
    x[9, 3] = np.nan
    layer = L.softmax_layer()
    y = layer.forward(L.DeviceMatrix.from_numpy(x, dtype=torch.float16)).to_numpy()
    ref = orc.softmax_fwd(f32(x))
    assert np.allclose(y[:, 0], 1.0 / h, rtol=2e-3)
    assert y[7, 1] == 1.0 and y[:, 1].sum() == 1.0
    assert y[5, 2] == 1.0 and y[:, 2].sum() == 1.0
    # a NaN in the column: the reference's output for that column is all zeros (non-normal results are flushed)
    assert (ref[:, 3] == 0).all() and (y[:, 3] == 0).all()


def test_softmax_f16_special_values_on_walked_rows(L):
    """The same columns among more rows than the device has compute units (a workgroup walks
    several rows there), each special column landing in a different position of the walk."""
    h, w = 32768, 600
    rng = np.random.default_rng(5)
    x = rand(rng, h, w, 0, 2).astype(np.float16)
    cols = {"equal": 3, "dominant": 258, "minus_inf": 301, "nan": 599}
    x[:, cols["equal"]] = 3.0
    x[7, cols["dominant"]] = 60000.0
    x[:, cols["minus_inf"]] = -np.inf
    x[5, cols["minus_inf"]] = 1.0
    x[9, cols["nan"]] = np.nan
    y = L.softmax_layer().forward(L.DeviceMatrix.from_numpy(x, dtype=torch.float16)).to_numpy()
    ref = orc.softmax_fwd(f32(x))
    assert np.allclose(f32(y[:, cols["equal"]]), 1.0 / h, rtol=2e-3)
    assert y[7, cols["dominant"]] == 1.0 and y[:, cols["dominant"]].sum() == 1.0
    assert y[5, cols["minus_inf"]] == 1.0 and y[:, cols["minus_inf"]].sum() == 1.0
    assert (ref[:, cols["nan"]] == 0).all() and (y[:, cols["nan"]] == 0).all()
    rest = [c for c in range(w) if c not in cols.values()]
    check("softmax f16 walked rows y", f32(y[:, rest]), f32(ref[:, rest]), tol=TOL_F16)
    ly = L.log_softmax_layer().forward(L.DeviceMatrix.from_numpy(x, dtype=torch.float16)).to_numpy()
    lref = orc.log_softmax_fwd(f32(x))
    check("log-softmax f16 walked rows y", f32(ly[:, rest]), f32(lref[:, rest]), tol=TOL_F16)
    assert np.all(np.isneginf(ly[:, cols["minus_inf"]][np.arange(h) != 5])) and abs(float(ly[5, cols["minus_inf"]])) == 0.0


@pytest.mark.parametrize("h", [70000, 50257])
def test_softmax_f16_special_values_on_long_rows(L, h):
    """Rows beyond the register kernels (two packed passes; 50257: cut at 16-byte boundaries)."""
    x = np.zeros((h, 5), dtype=np.float16)
    x[:, 0] = 3.0
    x[h - 2, 1] = 60000.0
    x[:, 2] = -np.inf
    x[5, 2] = 1.0
    x[9, 3] = np.nan
    x[:, 4] = -np.inf
    y = L.softmax_layer().forward(L.DeviceMatrix.from_numpy(x, dtype=torch.float16)).to_numpy()
    ref = orc.softmax_fwd(f32(x))
    assert np.allclose(f32(y[:, 0]), 1.0 / h, rtol=2e-3)
    assert y[h - 2, 1] == 1.0 and y[:, 1].sum() == 1.0
    assert y[5, 2] == 1.0 and y[:, 2].sum() == 1.0
    assert (ref[:, 3] == 0).all() and (y[:, 3] == 0).all()
    assert (ref[:, 4] == 0).all() and (y[:, 4] == 0).all()      # a column of -inf: 0 / 0, flushed


@pytest.mark.parametrize("kind", ["softmax", "log_softmax", "channelwise"])
@pytest.mark.parametrize("h,w,in_place", [(262144, 17, False), (65536, 40, False), (262144, 16, True), (131072, 31, True)])
def test_few_long_rows_all_in_flight(L, kind, h, w, in_place):
    """A handful of rows far longer than a workgroup holds, all resident at once: the cluster
    kernels with two rows per cluster (odd row counts leave the last cluster with one)."""
    rng = np.random.default_rng(h + 7 * w)
    x, dy = rand(rng, h, w, 0, 2), rand(rng, h, w)
    if kind == "channelwise":
        layer = L.channelwise_softmax_layer((2, h // 2))       # two windows per sample: 2 w rows of h / 2
        fwd = lambda a: orc.channelwise_softmax_fwd(a, 2, h // 2, h // 2)
        bwd = lambda y, g: orc.channelwise_softmax_bwd(y, g, 2, h // 2, h // 2)
    else:
        layer = L.softmax_layer() if kind == "softmax" else L.log_softmax_layer()
        fwd, bwd = _sm_oracle(kind)
    xm = L.DeviceMatrix.from_numpy(x)
    y = layer.forward(xm, in_place=in_place).to_numpy()
    check(f"{kind} few long rows y {h}x{w}", y, fwd(x), fwd(f64(x)))
    gm = L.DeviceMatrix.from_numpy(dy)
    dx = layer.backward(gm, in_place=in_place).to_numpy()
    check(f"{kind} few long rows dx {h}x{w}", dx, bwd(f32(y), dy), bwd(f64(y), f64(dy)))
    if kind != "log_softmax":
        assert np.abs(y.astype(np.float64).reshape(-1, (2 if kind == "channelwise" else 1) * w, order="F").sum(axis=0) - 1).max() < 1e-5


@pytest.mark.parametrize("kind", ["softmax", "log_softmax"])
@pytest.mark.parametrize("h,w,lds", [
    (50257, 6, (0, 0, 0, 0)),     # every tensor on the same frames: 16-byte access inside the rows
    (50257, 6, (0, 1, 2, 1)),     # leading dimensions that differ modulo 4: one float per access
    (50257, 6, (3, 7, 11, 3)),    # differ, but agree modulo 4: framed again
    (40002, 5, (1, 1, 1, 1)),     # even length, odd leading dimension
    (131071, 3, (0, 4, 0, 8)),
    # rows that fit one workgroup's registers: the same choice in the row kernels
    (16385, 5, (0, 1, 2, 1)), (16385, 5, (0, 4, 8, 0)), (30522, 4, (2, 2, 2, 2)), (8191, 70, (0, 0, 0, 0)),
    (32762, 3, (1, 1, 1, 1)), (32763, 3, (0, 0, 0, 0)),   # the longest frame of 8192 vectors, and one entry more
])
def test_long_rows_off_the_16_byte_grid(L, kind, h, w, lds):
    """Long rows that do not start on 16-byte boundaries: the kernels move them as 16-byte vectors
    between the rows' own first and last entries when x, y (and y, dy, dx) start every row at the
    same distance from a boundary, else float by float.  Padding rows hold NaN on the way in and
    must come back untouched."""
    rng = np.random.default_rng(h + sum(lds))
    x, dy = rand(rng, h, w, 0, 2), rand(rng, h, w)
    x[rng.integers(0, h, size=50), :] = 25.0
    fwd, bwd = _sm_oracle(kind)
    layer = L.softmax_layer() if kind == "softmax" else L.log_softmax_layer()
    pad_x, pad_y, pad_dy, pad_dx = lds
    layer.prev_activations = L.DeviceMatrix.from_numpy(x, ldim=h + pad_x)
    layer.activations = L.DeviceMatrix(h, w, ldim=h + pad_y, fill=-7.0)
    layer.fp_compute()
    y = layer.activations.to_numpy()
    check(f"{kind} off-grid y {h}x{w} {lds}", y, fwd(x), fwd(f64(x)))
    if pad_y:
        assert torch.all(layer.activations.tensor[:w, h:] == -7.0).item(), "wrote outside the rows"
    layer.prev_error_signals = L.DeviceMatrix.from_numpy(dy, ldim=h + pad_dy)
    layer.error_signals = L.DeviceMatrix(h, w, ldim=h + pad_dx, fill=-7.0)
    layer.bp_compute()
    dx = layer.error_signals.to_numpy()
    check(f"{kind} off-grid dx {h}x{w} {lds}", dx, bwd(f32(y), dy), bwd(f64(y), f64(dy)))
    if pad_dx:
        assert torch.all(layer.error_signals.tensor[:w, h:] == -7.0).item(), "wrote outside the rows"


@pytest.mark.parametrize("h", [16385, 50257])
@pytest.mark.parametrize("offsets", [(1, 1, 1, 1), (1, 2, 1, 1), (3, 3, 3, 3), (2, 0, 2, 0), (0, 0, 1, 0)])
def test_matrices_that_start_off_the_16_byte_grid(L, h, offsets):
    """Views into larger allocations: base pointers 4, 8 or 12 bytes past a 16-byte boundary.
    Tensors whose offsets agree take the 16-byte accesses, the others one float at a time; the
    floats in front of and behind every matrix must come back untouched."""
    w = 5
    ox, oy, ody, odx = offsets
    rng = np.random.default_rng(h + 7 * sum(offsets))
    x, dy = rand(rng, h, w, 0, 2), rand(rng, h, w)
    x[rng.integers(0, h, size=40), :] = 20.0
    capi = L.capi
    st = L._stream()

    def device(a, off):
        buf = torch.full((off + h * w + 8,), -7.0, device="cuda")
        if a is not None:
            buf[off:off + h * w] = torch.from_numpy(np.ascontiguousarray(a.T).reshape(-1)).cuda()
        return buf

    def host(buf, off):
        assert torch.all(buf[:off] == -7.0).item() and torch.all(buf[off + h * w:] == -7.0).item(), "wrote outside the matrix"
        return np.asfortranarray(buf[off:off + h * w].cpu().numpy().reshape(w, h).T)

    ptr = lambda buf, off: capi.vp(buf.data_ptr() + 4 * off)
    nb = capi.lib().lbn_softmax_workspace_bytes(h, w)
    ws = torch.zeros(max(nb, 64), dtype=torch.uint8, device="cuda")
    bx, by = device(x, ox), device(None, oy)
    capi.call("lbn_softmax_fwd_f32", st, h, w, ptr(bx, ox), h, ptr(by, oy), h, capi.vp(ws.data_ptr()), nb)
    y = host(by, oy)
    check(f"softmax off-grid base y {h} {offsets}", y, orc.softmax_fwd(x), orc.softmax_fwd(f64(x)))
    # backward reads the y it is given (offset oy), dy at ody, writes dx at odx
    bdy, bdx = device(dy, ody), device(None, odx)
    capi.call("lbn_softmax_bwd_f32", st, h, w, ptr(by, oy), h, ptr(bdy, ody), h, ptr(bdx, odx), h,
              capi.vp(ws.data_ptr()), nb)
    dx = host(bdx, odx)
    check(f"softmax off-grid base dx {h} {offsets}", dx, orc.softmax_bwd(f32(y), dy), orc.softmax_bwd(f64(y), f64(dy)))
    flag = capi.cint(0)
    capi.call("lbn_workspace_timed_out", st, capi.vp(ws.data_ptr()), flag)
    assert flag.value == 0


@pytest.mark.parametrize("kind", ["softmax", "log_softmax", "channelwise"])
@pytest.mark.parametrize("h,w", [(4096, 6), (777, 5), (70000, 2), (3003, 7)])
def test_softmax_family_in_place(L, kind, h, w):
    rng = np.random.default_rng(h + w)
    x, dy = rand(rng, h, w, 0, 2), rand(rng, h, w)
    if kind == "channelwise":
        C = 7 if h % 7 == 0 else 4
        layer = L.channelwise_softmax_layer((C, h // C))
        fwd = lambda a: orc.channelwise_softmax_fwd(a, C, h // C, h // C)
        bwd = lambda y, g: orc.channelwise_softmax_bwd(y, g, C, h // C, h // C)
    else:
        layer = L.softmax_layer() if kind == "softmax" else L.log_softmax_layer()
        fwd, bwd = _sm_oracle(kind)
    y_ref, y_ex = fwd(x), fwd(f64(x))
    xm = L.DeviceMatrix.from_numpy(x)
    ym = layer.forward(xm, in_place=True)
    assert ym is xm
    y = ym.to_numpy()
    check(f"{kind} in-place y", y, y_ref, y_ex, tol=TOL_F32)
    gm = L.DeviceMatrix.from_numpy(dy)
    dm = layer.backward(gm, in_place=True)
    assert dm is gm
    check(f"{kind} in-place dx", dm.to_numpy(), bwd(f32(y), dy), bwd(f64(y), f64(dy)))


def test_softmax_special_values(L):
    x = np.zeros((8, 5), dtype=np.float32, order="F")
    x[1, 0] = -95.0                       # denormal after exp -> flushed to 0 by softmax
    x[2, 0] = -200.0
    x[:, 1] = [50, -45, 50, -41, 0, 0, 0, 0]
    x[:, 2] = np.nan                      # NaN column -> all zeros (nothing is a normal float)
    x[:, 3] = -np.inf                     # max stays at -FLT_MAX, exp(-inf) = 0, 0 * inf = NaN -> 0
    x[3, 4] = np.inf                      # inf - inf = NaN at the maximum itself
    for kind, layer in (("softmax", L.softmax_layer()), ("log_softmax", L.log_softmax_layer())):
        y = layer.forward(L.DeviceMatrix.from_numpy(x)).to_numpy()
        ref = _sm_oracle(kind)[0](x)
        assert rel_err(y, ref) <= TOL_F32, kind
    # channelwise keeps denormals (no flush)
    xc = np.asfortranarray(x[:, :1])
    y = L.channelwise_softmax_layer((1, 8)).forward(L.DeviceMatrix.from_numpy(xc)).to_numpy()
    ref = orc.channelwise_softmax_fwd(xc, 1, 8, 8)
    assert 0 < y[1, 0] < np.finfo(np.float32).tiny
    assert rel_err(y, ref) <= TOL_F32


CWS_CASES = [
    # dims, dim, single_dim_mode, width
    ((5, 2, 7), 0, False, 15), ((5, 2, 7), -1, True, 15), ((64, 256), 0, False, 9),
    ((4, 8, 128), -1, True, 3), ((16, 4096), 0, False, 3), ((3, 40000), 0, False, 2),
    ((6, 10), 0, False, 4), ((12, 197, 197), -1, True, 3), ((5, 1001), 0, False, 6), ((3, 9001), 0, False, 2),
    ((16, 64, 64), -1, True, 8), ((512, 49), -1, True, 16), ((4096, 8), 0, False, 3),
]


@pytest.mark.parametrize("dims,dim,single,w", CWS_CASES)
def test_channelwise_softmax(L, dims, dim, single, w):
    rng = np.random.default_rng(sum(dims) + w)
    h = int(np.prod(dims))
    x, dy = rand(rng, h, w, 0.5, 1.0), rand(rng, h, w)
    layer = L.channelwise_softmax_layer(dims, dim=dim, single_dim_mode=single)
    cs, stride, C = layer.get_channel_size_and_stride()
    y = layer.forward(L.DeviceMatrix.from_numpy(x)).to_numpy()
    check("cws y", y, orc.channelwise_softmax_fwd(x, C, cs, stride), orc.channelwise_softmax_fwd(f64(x), C, cs, stride))
    dx = layer.backward(L.DeviceMatrix.from_numpy(dy)).to_numpy()
    check("cws dx", dx, orc.channelwise_softmax_bwd(f32(y), dy, C, cs, stride),
          orc.channelwise_softmax_bwd(f64(y), f64(dy), C, cs, stride))


# ===================================================================== layer norm
LN_CASES = [
    # dims, start_dim, width, affine, ld_pad
    ((1024,), 0, 128, True, 0), ((1024,), 0, 128, False, 0), ((256,), 0, 7, True, 0),
    ((64,), 0, 300, True, 0), ((4096,), 0, 40, True, 0), ((8192,), 0, 5, True, 0),
    ((16384,), 0, 3, True, 0), ((32768,), 0, 2, False, 0), ((40000,), 0, 2, True, 0),
    ((31,), 0, 15, True, 0), ((31, 2, 5), -1, 9, True, 0), ((31, 2, 5), 1, 9, True, 0),
    ((8, 512), -1, 33, True, 0), ((8, 512), 0, 6, True, 0), ((16, 64), 1, 700, True, 0),
    ((512,), 0, 6, True, 32), ((100,), 0, 6, True, 3), ((2048,), 0, 2000, True, 0),
    ((5, 1), -1, 4, False, 0),
    # backward plans: 512-thread teams with 32 entries per thread (masked and full), many
    # short rows (more than 256 persistent blocks), teams that leave threads idle
    ((12288,), 0, 5, True, 0), ((8192,), 0, 600, True, 0), ((768,), 0, 3000, True, 0),
    ((256,), 0, 70000, True, 0), ((5000,), 0, 40, True, 0),
    # rows longer than the register kernels hold: one 1024-thread workgroup per row, weight
    # gradients by row slabs (vector and scalar), groups, padded leading dimension
    ((150528,), 0, 6, True, 0), ((65536,), 0, 300, True, 0), ((4, 20000), -1, 9, True, 0),
    ((20001,), 0, 7, True, 0), ((20004,), 0, 5, True, 4), ((3, 224, 224), 0, 3, False, 0),
    # the same lengths on the 16-byte grid share a row among a cluster of workgroups: up to 128 members
    # (1048576 entries backward), beyond that the two-pass kernels again; more rows than clusters
    ((802816,), 0, 5, True, 0), ((1048576,), 0, 3, True, 0), ((1048580,), 0, 2, True, 0), ((32772,), 0, 700, True, 0),
    ((2, 100000), -1, 40, True, 8), ((50000,), 0, 33, False, 0),
    # rows of millions of entries: clusters that stream their share twice (forward; backward without weights)
    ((3000000,), 0, 3, False, 0), ((2500000,), 0, 2, True, 0), ((2, 2200000), -1, 2, False, 4), ((9000000,), 0, 1, False, 0),
    # rows off the 16-byte grid: the register kernels with one float per access
    ((1001,), 0, 40, True, 0), ((197, 769), -1, 3, True, 0), ((4095,), 0, 9, True, 0), ((4097,), 0, 9, True, 0),
    ((8191,), 0, 5, False, 0), ((49,), 0, 3000, True, 0), ((1000,), 0, 17, True, 3), ((7,), 0, 100000, True, 0),
    # longer rows off the 16-byte grid: two passes of 16-byte accesses at 4-byte alignment, every n % 4
    ((10001,), 0, 7, True, 0), ((50001,), 0, 5, False, 0), ((50002,), 0, 3, True, 1), ((30003,), 0, 4, True, 0),
    ((3, 89401), -1, 3, False, 0), ((20000,), 0, 6, True, 1), ((1,), 0, 70000, True, 0),
    # many short rows: teams of 16 lanes, four rows per wave
    ((1024, 64), -1, 8, True, 0), ((512, 128), -1, 16, True, 0), ((64, 256), -1, 70, True, 0), ((4099, 16), -1, 3, False, 0),
    ((49,), 0, 5000, True, 0), ((600, 20), -1, 9, True, 0), ((4096, 8), -1, 1, True, 0), ((2048, 12), -1, 2, True, 4),
    # calls that move more than the last-level cache holds (192 MiB tensors): streaming loads
    ((4096,), 0, 12288, True, 0), ((12288, 64), -1, 64, False, 0),
]


def _ln_run(L, x, dy, dims, start_dim, affine, pad, scale, bias, mode=None, tol=TOL_F32, half=False):
    h, w = x.shape
    kw = dict(scale_values=scale, bias_values=bias) if affine else {}
    if mode is not None:
        kw["stats_mode"] = mode
    layer = L.layer_norm_layer(dims, 1e-5, affine, affine, start_dim, **kw)
    G, n = layer.num_normalized, layer.normalization_size
    tdt = torch.float16 if half else torch.float32
    y = layer.forward(L.DeviceMatrix.from_numpy(x, dtype=tdt, ldim=h + pad)).to_numpy()
    stats = layer.m_statistics.to_numpy()
    dx = layer.backward(L.DeviceMatrix.from_numpy(dy, dtype=tdt, ldim=h + pad)).to_numpy()
    sgrad = layer.m_statistics_gradient.to_numpy()
    out = dict(y=y, stats=stats, dx=dx, sgrad=sgrad)
    if affine:
        out["dscale"] = layer.m_scale_gradient.to_numpy()
        out["dbias"] = layer.m_bias_gradient.to_numpy()
    g = scale if affine else None
    b = bias if affine else None
    ref, ex = {}, {}
    for dst, conv in ((ref, f32), (ex, f64)):
        xx, gg = conv(x), conv(dy)
        sc = None if g is None else conv(g)
        bi = None if b is None else conv(b)
        dst["y"], dst["stats"] = orc.layer_norm_fwd(xx, G, n, n, 1e-5, sc, bi)
        dst["dx"], dst["sgrad"], dst["dscale"], dst["dbias"] = orc.layer_norm_bwd(
            xx, gg, dst["stats"], G, n, n, 1e-5, sc, affine, affine)
    if n <= 1:
        out.pop("sgrad"); ref.pop("sgrad")   # left untouched by the reference in this case
    res = {}
    for k in out:
        res[k] = check(f"layer_norm {k} dims={dims} w={w}", out[k], ref[k], ex[k], tol=tol)
    return res


@pytest.mark.parametrize("dims,start_dim,w,affine,pad", LN_CASES)
def test_layer_norm_f32(L, dims, start_dim, w, affine, pad):
    rng = np.random.default_rng(int(np.prod(dims)) + w)
    h = int(np.prod(dims))
    x, dy = rand(rng, h, w, 0.3, 1.5), rand(rng, h, w)
    n = int(np.prod(dims[(start_dim if start_dim >= 0 else len(dims) + start_dim):]))
    scale = (1 + 0.3 * rng.standard_normal(n)).astype(np.float32)
    bias = (0.3 * rng.standard_normal(n)).astype(np.float32)
    _ln_run(L, x, dy, dims, start_dim, affine, pad, scale, bias)


@pytest.mark.parametrize("dims,start_dim,w", [((1024,), 0, 64), ((31,), 0, 15), ((8, 512), -1, 9), ((40000,), 0, 4)])
def test_layer_norm_reference_formula_mode(L, dims, start_dim, w):
    """E[x^2]-mean^2 mode reproduces the reference's variance, clamp included."""
    rng = np.random.default_rng(5)
    h = int(np.prod(dims))
    x, dy = rand(rng, h, w, 3.0, 0.5), rand(rng, h, w)
    x[:, 0] = 7.0   # constant column: the clamp at zero decides the variance
    _ln_run(L, x, dy, dims, start_dim, False, 0, None, None, mode=L.LBN_STATS_SUMSQ)


@pytest.mark.parametrize("dims,start_dim,w,pad", [((4096,), 0, 64, 0), ((512,), 0, 100, 0), ((64,), 0, 9, 0),
                                                   ((8, 1024), -1, 5, 0), ((100,), 0, 7, 0), ((2048,), 0, 600, 8),
                                                   ((16384,), 0, 3, 0), ((16384,), 0, 40, 0), ((8192,), 0, 300, 0),
                                                   ((768,), 0, 1000, 0), ((12288,), 0, 9, 0), ((12288,), 0, 600, 0), ((10248,), 0, 520, 8),
                                                   ((32768,), 0, 20, 0), ((150528,), 0, 3, 0), ((20000,), 0, 5, 8),
                                                   ((1024, 256), -1, 8, 0), ((512, 64), -1, 16, 0), ((128, 512), -1, 40, 0),
                                                   # even lengths that are not a multiple of 8: one pair per access
                                                   ((4100,), 0, 40, 0), ((1002,), 0, 33, 0), ((6, 770), -1, 9, 0),
                                                   ((8190,), 0, 5, 2), ((16382,), 0, 3, 0), ((4100, 12), -1, 2, 0),
                                                   ((1001,), 0, 7, 0), ((4099,), 0, 9, 0), ((10001,), 0, 5, 1), ((513,), 0, 40, 0),   # odd: eight entries per access at 2-byte alignment
                                                   ((50003,), 0, 3, 0), ((20002,), 0, 4, 1), ((301,), 0, 20, 0),
                                                   # long rows shared by clusters of workgroups
                                                   ((802816,), 0, 4, 0), ((65536,), 0, 150, 0), ((2, 100000), -1, 20, 8),
                                                   ((1048576,), 0, 2, 0), ((5000000,), 0, 2, 0),
                                                   ((8192,), 0, 12288, 0)])   # 192 MiB tensors: streaming loads
def test_layer_norm_f16(L, dims, start_dim, w, pad):
    rng = np.random.default_rng(int(np.prod(dims)) * 3 + w)
    h = int(np.prod(dims))
    x = rand(rng, h, w, 0.3, 1.5).astype(np.float16).astype(np.float32)
    dy = rand(rng, h, w).astype(np.float16).astype(np.float32)
    n = int(np.prod(dims[(start_dim if start_dim >= 0 else len(dims) + start_dim):]))
    scale = (1 + 0.1 * rng.standard_normal(n)).astype(np.float32)
    bias = (0.1 * rng.standard_normal(n)).astype(np.float32)
    _ln_run(L, x, dy, dims, start_dim, True, pad, scale, bias, tol=TOL_F16, half=True)


@pytest.mark.parametrize("affine,mode", [(False, None), (True, None), (True, "sumsq")])
@pytest.mark.parametrize("dims,start_dim,w,pad", [
    ((9,), 0, 11, 0), ((15,), 0, 300, 0), ((17,), 0, 5000, 0), ((63,), 0, 40, 0), ((65,), 0, 4100, 0),
    ((129,), 0, 33, 0), ((255,), 0, 4200, 0), ((257,), 0, 700, 0), ((511,), 0, 64, 0), ((1023,), 0, 9, 0),
    ((1025,), 0, 70, 0), ((2047,), 0, 12, 0), ((2049,), 0, 300, 0), ((3001,), 0, 17, 0), ((4095,), 0, 5, 0),
    ((4097,), 0, 40, 0), ((8191,), 0, 6, 0), ((16385,), 0, 7, 0), ((24001,), 0, 3, 0), ((32767,), 0, 4, 0),
    ((6, 771), -1, 9, 0), ((3, 35), -1, 2000, 0),
    # whole eights of entries behind odd leading dimensions: no partial vector, still unaligned
    ((1024,), 0, 9, 1), ((64,), 0, 5000, 3), ((2048,), 0, 33, 5)])
def test_layer_norm_f16_unaligned_rows(L, dims, start_dim, w, pad, affine, mode):
    """fp16 rows that are not whole aligned vectors, in 16-byte accesses at 2-byte alignment: the row's
    last n % 8 entries come from a vector that overlaps its neighbour."""
    rng = np.random.default_rng(int(np.prod(dims)) * 11 + w + pad)
    h = int(np.prod(dims))
    x = rand(rng, h, w, 0.3, 1.5).astype(np.float16).astype(np.float32)
    dy = rand(rng, h, w).astype(np.float16).astype(np.float32)
    n = int(np.prod(dims[(start_dim if start_dim >= 0 else len(dims) + start_dim):]))
    scale = (1 + 0.1 * rng.standard_normal(n)).astype(np.float32)
    bias = (0.1 * rng.standard_normal(n)).astype(np.float32)
    _ln_run(L, x, dy, dims, start_dim, affine, pad, scale, bias, tol=TOL_F16, half=True,
            mode=L.LBN_STATS_SUMSQ if mode else None)


@pytest.mark.parametrize("affine,mode", [(False, None), (True, None), (True, "sumsq")])
@pytest.mark.parametrize("dims,start_dim,w,pad", [
    ((5,), 0, 4100, 0), ((7,), 0, 9000, 1), ((35,), 0, 5000, 0), ((127,), 0, 4200, 0), ((126,), 0, 4100, 1),
    ((2049,), 0, 70, 0), ((3001,), 0, 9, 0), ((4099,), 0, 33, 0), ((8191,), 0, 6, 0), ((10001,), 0, 12, 0),
    ((12290,), 0, 5, 0), ((16383,), 0, 3, 0), ((16385,), 0, 3, 0), ((30001,), 0, 4, 0), ((32769,), 0, 2, 0),
    ((3, 2731), -1, 9, 0), ((4, 33), -1, 1500, 0),
    # whole fours of entries behind leading dimensions that are not: no partial vector, still unaligned
    ((4096,), 0, 9, 1), ((64,), 0, 5000, 3), ((12288,), 0, 7, 2)])
def test_layer_norm_f32_unaligned_rows(L, dims, start_dim, w, pad, affine, mode):
    """fp32 rows that are not whole aligned vectors, in 16-byte accesses at 4-byte alignment: the row's
    last n % 4 entries come from a vector that overlaps its neighbour."""
    rng = np.random.default_rng(int(np.prod(dims)) * 13 + w + pad)
    h = int(np.prod(dims))
    x, dy = rand(rng, h, w, 0.3, 1.5), rand(rng, h, w)
    n = int(np.prod(dims[(start_dim if start_dim >= 0 else len(dims) + start_dim):]))
    scale = (1 + 0.3 * rng.standard_normal(n)).astype(np.float32)
    bias = (0.3 * rng.standard_normal(n)).astype(np.float32)
    _ln_run(L, x, dy, dims, start_dim, affine, pad, scale, bias, mode=L.LBN_STATS_SUMSQ if mode else None)


# ===================================================================== instance norm
@pytest.mark.parametrize("dims,w,pad", [((5, 3, 7), 15, 0), ((64, 56, 56), 6, 0), ((8, 1024), 33, 0),
                                        ((2, 1048576), 2, 0), ((4, 96, 96, 96), 3, 0),   # volumes: clusters of workgroups per channel
                                        ((2, 160, 160, 160), 1, 0), ((3, 2500000), 2, 4),   # streaming clusters
                                        ((3, 50000), 40, 4),
                                        ((3, 100000), 2, 0), ((7, 1), 5, 0), ((16, 31), 40, 4),
                                        ((256, 16, 16), 64, 0), ((3, 224, 224), 8, 0), ((2, 64, 64, 64), 2, 0),
                                        ((256, 7, 7), 32, 0), ((64, 3, 3), 9, 0), ((5, 4097), 6, 0),
                                        ((256, 8, 8), 32, 0), ((512, 4, 4), 16, 0), ((64, 16, 16), 70, 0),
                                        ((3, 299, 299), 5, 0), ((2, 111, 111), 9, 1), ((1024, 1), 300, 0)])
def test_instance_norm(L, dims, w, pad):
    rng = np.random.default_rng(int(np.prod(dims)) + 7 * w)
    h = int(np.prod(dims))
    C, cs = dims[0], h // dims[0]
    x, dy = rand(rng, h, w, 0.5, 2.0), rand(rng, h, w)
    layer = L.instance_norm_layer(dims, 1e-5)
    y = layer.forward(L.DeviceMatrix.from_numpy(x, ldim=h + pad)).to_numpy()
    dx = layer.backward(L.DeviceMatrix.from_numpy(dy, ldim=h + pad)).to_numpy()
    y32, s32 = orc.instance_norm_fwd(f32(x), C, cs, 1e-5)
    y64, s64 = orc.instance_norm_fwd(f64(x), C, cs, 1e-5)
    check(f"instance_norm y dims={dims}", y, y32, y64)
    check(f"instance_norm dx dims={dims}", dx, orc.instance_norm_bwd(f32(x), f32(dy), s32, C, cs, 1e-5),
          orc.instance_norm_bwd(f64(x), f64(dy), s64, C, cs, 1e-5))


# ===================================================================== entry-wise batch norm
@pytest.mark.parametrize("h,w,pad", [(105, 14, 0), (105, 29, 0), (4096, 64, 0), (4096, 256, 0), (1024, 300, 0),
                                     (200000, 16, 0), (64, 1, 0), (260, 7, 4), (258, 9, 0), (100000, 33, 0),
                                     (2048, 1000, 0), (8196, 257, 4), (60, 513, 0),   # wider than the register tiles
                                     (4096, 1024, 0), (512, 4100, 0), (64, 5000, 4), (1000, 1777, 0), (4, 2000, 0), (4096, 1023, 0),   # column slabs from 1024 columns
                                     (786432, 64, 0)])   # 192 MiB tensors: streaming loads
def test_entrywise_batch_norm(L, h, w, pad):
    rng = np.random.default_rng(h + 3 * w)
    x, dy = rand(rng, h, w, 0.5, 2.0), rand(rng, h, w)
    rm0 = rng.normal(size=h).astype(np.float32)
    rv0 = rng.uniform(0.5, 2.0, size=h).astype(np.float32)

    def oracle(conv, training):
        rm, rv = conv(rm0).copy(), conv(rv0).copy()
        y, st = orc.entrywise_batch_norm_fwd(conv(x), 0.9, 1e-5, rm, rv, training)
        dx, sg = orc.entrywise_batch_norm_bwd(conv(x), conv(dy), st, 1e-5, rv, training)
        return dict(y=y, stats=st, dx=dx, sgrad=sg, rmean=rm, rvar=rv)

    for training in (True, False):
        layer = L.entrywise_batch_normalization_layer((h,), 0.9, 1e-5)
        layer.weights[0].tensor.copy_(torch.from_numpy(rm0))
        layer.weights[1].tensor.copy_(torch.from_numpy(rv0))
        layer.training = training
        y = layer.forward(L.DeviceMatrix.from_numpy(x, ldim=h + pad)).to_numpy()
        dx = layer.backward(L.DeviceMatrix.from_numpy(dy, ldim=h + pad)).to_numpy()
        got = dict(y=y, dx=dx, rmean=layer.weights[0].to_numpy(), rvar=layer.weights[1].to_numpy())
        if training:
            got["stats"] = layer.m_batch_statistics.to_numpy()
            if w > 1:
                got["sgrad"] = layer.m_batch_statistics_gradient.to_numpy()
        r32, r64 = oracle(f32, training), oracle(f64, training)
        for k in got:
            check(f"entrywise_bn {k} h={h} w={w} training={training}", got[k], r32[k], r64[k])


def test_entrywise_batch_norm_clamps_negative_variance(L):
    """Where the reference's fp32 E[x^2] - mean^2 is negative (tests/test_oracle.py pins that
    it keeps -2 and returns NaN), both GPU paths clamp the variance at zero: y is finite."""
    from lbann_amd import capi
    x = f32(np.array([[3198.374755859375, 3198.375], [1.0, 3.0], [0.5, -0.5], [2.0, 2.0]], dtype=np.float32))
    layer = L.entrywise_batch_normalization_layer((4,), 0.9, 1e-5)
    y = layer.forward(L.DeviceMatrix.from_numpy(x)).to_numpy()
    stats = layer.m_batch_statistics.to_numpy()
    assert np.isfinite(y).all() and stats[0, 1] >= 0.0
    assert stats[1, 1] == np.float32(2.0)
    # the split statistics step on the reference's own sums: same clamp
    xd = L.DeviceMatrix.from_numpy(x)
    st = L.DeviceMatrix(4, 2)
    rm, rv = L._Vector(4, "cuda", np.zeros(4)), L._Vector(4, "cuda", np.ones(4))
    s = capi.vp(torch.cuda.current_stream().cuda_stream)
    L.call("lbn_entrywise_batch_norm_fwd_sums_f32", s, 4, 2, xd.Buffer(), xd.ldim, st.Buffer(), st.ldim)
    L.call("lbn_entrywise_batch_norm_fwd_stats_f32", s, 4, 2, 0.9, st.Buffer(), st.ldim, rm.Buffer(), rv.Buffer())
    split = st.to_numpy()
    assert split[0, 1] == 0.0 and split[1, 1] == np.float32(2.0)


@pytest.mark.parametrize("h,w,w0,pad", [(105, 29, 14, 0), (4096, 64, 32, 0), (1024, 300, 7, 0), (260, 7, 3, 4),
                                        (258, 9, 9, 0), (100000, 33, 16, 0), (8196, 257, 200, 4), (60, 513, 512, 0),
                                        (64, 1, 1, 0), (64, 2, 1, 0)])
def test_entrywise_batch_norm_split_over_two_ranks(L, h, w, w0, pad):
    """The mini-batch's columns [0, w0) on one rank and [w0, w) on another: local sums, their
    sum in place of the all-reduce, statistics with the global count, apply per rank; the
    same for backward.  Together the two ranks must give what the reference gives on the
    whole mini-batch (entrywise_batch_normalization.cpp:97-100, :301-303)."""
    from lbann_amd import capi
    rng = np.random.default_rng(h + 5 * w)
    x, dy = rand(rng, h, w, 0.5, 2.0), rand(rng, h, w)
    rm0 = rng.normal(size=h).astype(np.float32)
    rv0 = rng.uniform(0.5, 2.0, size=h).astype(np.float32)
    st = capi.vp(torch.cuda.current_stream().cuda_stream)
    p = lambda t: capi.vp(t.data_ptr())
    parts = [(0, w0), (w0, w)]
    xs = [L.DeviceMatrix.from_numpy(x[:, a:b], ldim=h + pad) for a, b in parts]
    gs = [L.DeviceMatrix.from_numpy(dy[:, a:b], ldim=h + pad) for a, b in parts]
    ys = [L.DeviceMatrix(h, b - a, ldim=h + pad, fill=float("nan")) for a, b in parts]
    ds = [L.DeviceMatrix(h, b - a, ldim=h + pad, fill=float("nan")) for a, b in parts]
    ldst = h + pad

    def oracle(conv):
        rm, rv = conv(rm0).copy(), conv(rv0).copy()
        y, stt = orc.entrywise_batch_norm_fwd(conv(x), 0.9, 1e-5, rm, rv, True)
        dx, sg = orc.entrywise_batch_norm_bwd(conv(x), conv(dy), stt, 1e-5, rv, True)
        return dict(y=y, stats=stt, dx=dx, sgrad=sg, rmean=rm, rvar=rv)

    # forward: sums per rank -> "all-reduce" -> statistics (the same on both ranks) -> apply
    local = [L.DeviceMatrix(h, 2, ldim=ldst, fill=float("nan")) for _ in parts]
    for m, xm in zip(local, xs):
        capi.call("lbn_entrywise_batch_norm_fwd_sums_f32", st, h, xm.width, xm.Buffer(), xm.ldim, m.Buffer(), m.ldim)
    sums = local[0].to_numpy().astype(np.float64)
    assert rel_err(sums[:, 0], x[:, :w0].astype(np.float64).sum(axis=1)) < 1e-5
    assert rel_err(sums[:, 1], (x[:, :w0].astype(np.float64) ** 2).sum(axis=1)) < 1e-5
    stats = L.DeviceMatrix(h, 2, ldim=ldst)
    stats.tensor[:, :h] = local[0].tensor[:, :h] + local[1].tensor[:, :h]
    rm, rv = torch.from_numpy(rm0).cuda(), torch.from_numpy(rv0).cuda()
    capi.call("lbn_entrywise_batch_norm_fwd_stats_f32", st, h, w, 0.9, stats.Buffer(), stats.ldim, p(rm), p(rv))
    mean_ptr = stats.Buffer()
    var_ptr = capi.vp(stats.tensor.data_ptr() + 4 * stats.ldim)
    for xm, ym in zip(xs, ys):
        capi.call("lbn_entrywise_batch_norm_fwd_apply_f32", st, h, xm.width, 1e-5, xm.Buffer(), xm.ldim, ym.Buffer(),
                  ym.ldim, mean_ptr, var_ptr)
    # backward
    glocal = [L.DeviceMatrix(h, 2, ldim=ldst, fill=float("nan")) for _ in parts]
    for m, xm, gm in zip(glocal, xs, gs):
        capi.call("lbn_entrywise_batch_norm_bwd_sums_f32", st, h, xm.width, 1e-5, xm.Buffer(), xm.ldim, gm.Buffer(),
                  gm.ldim, stats.Buffer(), stats.ldim, m.Buffer(), m.ldim)
    sgrad = L.DeviceMatrix(h, 2, ldim=ldst)
    sgrad.tensor[:, :h] = glocal[0].tensor[:, :h] + glocal[1].tensor[:, :h]
    for xm, gm, dm in zip(xs, gs, ds):
        capi.call("lbn_entrywise_batch_norm_bwd_apply_f32", st, h, xm.width, w, 1e-5, xm.Buffer(), xm.ldim, gm.Buffer(),
                  gm.ldim, dm.Buffer(), dm.ldim, stats.Buffer(), stats.ldim, sgrad.Buffer(), sgrad.ldim)
    got = dict(y=np.concatenate([m.to_numpy() for m in ys], axis=1), stats=stats.to_numpy(),
               dx=np.concatenate([m.to_numpy() for m in ds], axis=1), rmean=rm.cpu().numpy(), rvar=rv.cpu().numpy())
    if w > 1:
        got["sgrad"] = sgrad.to_numpy()
    r32, r64 = oracle(f32), oracle(f64)
    for k in got:
        check(f"entrywise_bn split {k} h={h} w={w} w0={w0}", got[k], r32[k], r64[k])
    if pad:
        assert torch.isnan(ys[0].tensor[:, h:]).all() and torch.isnan(ds[0].tensor[:, h:]).all()
    # inference: apply with the running statistics equals the unsplit call's inference mode
    ym = L.DeviceMatrix(h, xs[0].width, ldim=h + pad)
    rm_i, rv_i = torch.from_numpy(rm0).cuda(), torch.from_numpy(rv0).cuda()
    capi.call("lbn_entrywise_batch_norm_fwd_apply_f32", st, h, xs[0].width, 1e-5, xs[0].Buffer(), xs[0].ldim, ym.Buffer(),
              ym.ldim, p(rm_i), p(rv_i))
    y_inf, _ = orc.entrywise_batch_norm_fwd(f32(x[:, :w0]), 0.9, 1e-5, rm0.copy(), rv0.copy(), False)
    check("entrywise_bn split inference y", ym.to_numpy(), y_inf)


def test_entrywise_batch_norm_layer_with_allreduce_hook(L):
    """The layer mirror with a collective: two layer objects (ranks) hold 20 and 13 columns of
    one mini-batch; the hook adds what the other rank computed, as comm.allreduce would."""
    rng = np.random.default_rng(97)
    h, w, w0 = 1000, 33, 20
    x, dy = rand(rng, h, w, -0.3, 1.5), rand(rng, h, w)
    halves = [(0, w0), (w0, w)]
    # lock-step emulation: rank 1's local sums are computed first through the C ABI
    # and handed to rank 0's hook, then the other way round
    from lbann_amd import capi
    st = capi.vp(torch.cuda.current_stream().cuda_stream)
    mats = [L.DeviceMatrix.from_numpy(x[:, a:b]) for a, b in halves]
    gmats = [L.DeviceMatrix.from_numpy(dy[:, a:b]) for a, b in halves]
    results = []
    for me, other in ((0, 1), (1, 0)):
        phase = {"n": 0}

        def hook(m, me=me, other=other, phase=phase):
            peer = L.DeviceMatrix(h, 2)
            if phase["n"] == 0:
                capi.call("lbn_entrywise_batch_norm_fwd_sums_f32", st, h, mats[other].width, mats[other].Buffer(),
                          mats[other].ldim, peer.Buffer(), peer.ldim)
            else:
                capi.call("lbn_entrywise_batch_norm_bwd_sums_f32", st, h, mats[other].width, 1e-5, mats[other].Buffer(),
                          mats[other].ldim, gmats[other].Buffer(), gmats[other].ldim, layer.m_batch_statistics.Buffer(),
                          layer.m_batch_statistics.ldim, peer.Buffer(), peer.ldim)
            m.tensor[:, :h] += peer.tensor[:, :h]
            phase["n"] += 1

        layer = L.entrywise_batch_normalization_layer((h,), 0.9, 1e-5, comm_allreduce=hook, statistics_count=w)
        y = layer.forward(mats[me]).to_numpy()
        dx = layer.backward(gmats[me]).to_numpy()
        assert phase["n"] == 2
        results.append((y, dx, layer.m_batch_statistics.to_numpy(), layer.weights[0].to_numpy(), layer.weights[1].to_numpy()))
    rm, rv = np.zeros(h, np.float32), np.ones(h, np.float32)
    y_ref, st_ref = orc.entrywise_batch_norm_fwd(x, 0.9, 1e-5, rm, rv, True)
    dx_ref, _ = orc.entrywise_batch_norm_bwd(x, dy, st_ref, 1e-5, rv, True)
    x64, dy64 = f64(x), f64(dy)
    y64, st64 = orc.entrywise_batch_norm_fwd(x64, 0.9, 1e-5, np.zeros(h), np.ones(h), True)
    dx64, _ = orc.entrywise_batch_norm_bwd(x64, dy64, st64, 1e-5, np.ones(h), True)
    check("hooked entrywise_bn y", np.concatenate([r[0] for r in results], axis=1), y_ref, y64)
    check("hooked entrywise_bn dx", np.concatenate([r[1] for r in results], axis=1), dx_ref, dx64)
    for r in results:
        check("hooked entrywise_bn stats", r[2], st_ref, st64)
        check("hooked entrywise_bn running mean", r[3], rm)
        check("hooked entrywise_bn running var", r[4], rv)
    # inference through the hooked layer: running statistics, no collective
    layer.training = False
    y_inf = layer.forward(mats[1]).to_numpy()
    y_inf_ref, _ = orc.entrywise_batch_norm_fwd(f32(x[:, w0:]), 0.9, 1e-5, rm.copy(), rv.copy(), False)
    check("hooked entrywise_bn inference", y_inf, y_inf_ref)


def test_entrywise_batch_norm_split_empty_and_rejected_arguments(L):
    from lbann_amd import capi
    st = capi.vp(torch.cuda.current_stream().cuda_stream)
    null = capi.vp(None)
    lib = capi.lib()
    buf = torch.full((4096,), 3.0, device="cuda")
    p = capi.vp(buf.data_ptr())
    # a rank without local columns contributes zero sums
    assert lib.lbn_entrywise_batch_norm_fwd_sums_f32(st, 16, 0, null, 16, p, 16) == 0
    assert lib.lbn_entrywise_batch_norm_bwd_sums_f32(st, 10, 0, 1e-5, null, 10, null, 10, p, 2048, capi.vp(buf.data_ptr() + 4 * 64), 10) == 0
    torch.cuda.synchronize()
    assert buf[:32].abs().sum().item() == 0.0 and buf[32].item() == 3.0
    assert buf[64:84].abs().sum().item() == 0.0 and buf[84].item() == 3.0
    assert lib.lbn_entrywise_batch_norm_fwd_sums_f32(st, 0, 4, null, 1, null, 1) == 0
    assert lib.lbn_entrywise_batch_norm_fwd_apply_f32(st, 8, 0, 1e-5, null, 8, null, 8, null, null) == 0
    # a single sample in the whole mini-batch: variance 1, running statistics untouched, dx = 0
    buf.fill_(3.0)
    run = torch.full((16,), 5.0, device="cuda")
    assert lib.lbn_entrywise_batch_norm_fwd_stats_f32(st, 8, 1, 0.9, p, 8, capi.vp(run.data_ptr()), capi.vp(run.data_ptr() + 32)) == 0
    assert lib.lbn_entrywise_batch_norm_bwd_apply_f32(st, 8, 1, 1, 1e-5, null, 8, null, 8, capi.vp(buf.data_ptr() + 4 * 100), 8, null, 8, null, 8) == 0
    torch.cuda.synchronize()
    assert buf[:8].tolist() == [3.0] * 8 and buf[8:16].tolist() == [1.0] * 8 and (run == 5.0).all()
    assert buf[100:108].abs().sum().item() == 0.0 and buf[108].item() == 3.0
    # rejected
    E = capi.LBN_ERR_INVALID_ARGUMENT
    assert lib.lbn_entrywise_batch_norm_fwd_sums_f32(st, 8, 4, p, 4, p, 8) == E
    assert lib.lbn_entrywise_batch_norm_fwd_sums_f32(st, 8, 4, p, 8, p, 4) == E
    assert lib.lbn_entrywise_batch_norm_fwd_sums_f32(st, 8, 4, null, 8, p, 8) == E
    assert lib.lbn_entrywise_batch_norm_fwd_stats_f32(st, 8, 4, 0.9, p, 8, null, p) == E
    assert lib.lbn_entrywise_batch_norm_fwd_apply_f32(st, 8, 4, 1e-5, p, 8, p, 8, null, p) == E
    assert lib.lbn_entrywise_batch_norm_bwd_sums_f32(st, 8, 4, 1e-5, p, 8, p, 8, p, 8, null, 8) == E
    assert lib.lbn_entrywise_batch_norm_bwd_apply_f32(st, 8, 4, 4, 1e-5, p, 8, p, 8, null, 8, p, 8, p, 8) == E
    assert lib.lbn_entrywise_batch_norm_bwd_apply_f32(st, 8, 4, 4, 1e-5, p, 8, p, 8, p, 8, p, 4, p, 8) == E
    torch.cuda.synchronize()


# ===================================================================== batch norm
BN_CASES = [
    # dims (C, ...), width, bessel, ld_pad
    ((7, 5, 3), 14, True, 0), ((7, 5, 3), 29, False, 0), ((8, 16, 16), 12, True, 0),
    ((256, 4, 4), 32, True, 0), ((3, 56, 56), 16, True, 0), ((16, 28, 28), 8, False, 0),
    ((5, 12), 10, True, 4), ((5, 13), 10, True, 0), ((2, 1), 1, True, 0), ((1, 100000), 3, True, 0),
    ((70, 1), 50, True, 0), ((70000, 1), 3, True, 0),   # more channels than gridDim.y could hold
    # channels that are not whole 16-byte vectors on a quad-aligned matrix: row-tile kernels
    ((2048, 7, 7), 16, True, 0), ((4096,), 64, True, 0), ((64, 7, 7), 300, False, 0), ((12, 3, 3), 20, True, 0),
    ((8, 5), 7, True, 4), ((4, 1), 1, True, 0), ((1024, 1), 2048, True, 0),
    ((512, 2, 2), 40, True, 0), ((300, 8), 33, False, 0), ((64, 4), 700, True, 4),   # one or two vectors per channel
    ((8, 55, 55), 300, True, 0), ((4, 111, 111), 20, False, 0), ((12, 27, 27), 400, True, 4),   # odd maps of many rows: a workgroup merges a channel
    # register-resident row tiles (w <= 256): 64-row and 256-row layouts, every columns-per-thread count
    ((4096,), 5, True, 0), ((4096,), 30, True, 0), ((1024, 1), 100, True, 0), ((2000, 2), 200, False, 0),
    ((333, 4), 256, True, 0), ((128, 7, 7), 3, True, 0), ((128, 7, 7), 10, True, 0), ((64, 7, 7), 24, True, 0),
    ((64, 7, 7), 40, False, 0), ((32, 7, 7), 64, True, 4), ((40, 5, 5), 50, True, 0), ((16, 3, 3), 250, True, 0),
    ((256, 4, 4), 200, True, 0), ((100, 12), 64, True, 0),
    # more channels than resident clusters: some clusters take two or three channels in turn, others one
    ((478, 16), 577, True, 0), ((1500, 4, 4), 600, False, 0), ((900, 64), 300, True, 0),
    # many channels of 512 to 8192 vectors: one workgroup keeps a channel (256, 512 and 1024 threads)
    ((1024, 14, 14), 32, True, 0), ((600, 8, 8), 100, False, 4), ((300, 28, 28), 40, True, 0), ((2048, 4, 4), 130, True, 0),
    ((1100, 8), 300, False, 0), ((520, 14, 14), 72, True, 0),
    # the same for channels that are not whole 16-byte vectors (7 x 7 maps): single floats, up to 16 per thread
    ((2048, 7, 7), 128, True, 0), ((512, 7, 7), 256, False, 0), ((300, 5, 5), 100, True, 0), ((256, 3, 3), 200, True, 3),
    ((1024, 1), 1100, True, 1), ((130, 7, 7), 300, True, 0),
    # channels of up to a million entries: clusters of more than 64 workgroups (two slots per polling lane)
    ((3, 56, 56), 256, True, 0), ((2, 802816), 1, True, 0), ((2, 1000000), 1, False, 0), ((1, 1100000), 1, True, 0),
    # beyond that: clusters that stream their share twice (backward from 1 M entries, forward from 2 M)
    ((3, 112, 112), 256, True, 0), ((2, 2400000), 1, False, 0), ((5, 1300000), 2, True, 4), ((1, 6000000), 1, True, 0),
]


def _bn_run(L, x, dy, dims, bessel, pad, scale, bias, mode=None, training=True, half=False):
    h, w = x.shape
    C = dims[0]
    cs = h // C
    kw = {} if mode is None else {"stats_mode": mode}
    layer = L.batch_normalization_layer(dims, 0.9, 1e-5, bessel, scale, bias, **kw)
    layer.training = training
    rm0 = (0.1 * np.arange(C)).astype(np.float32)
    rv0 = (1.0 + 0.05 * np.arange(C)).astype(np.float32)
    layer.weights[2].tensor[:C] = torch.from_numpy(rm0).cuda()
    layer.weights[3].tensor[:C] = torch.from_numpy(rv0).cuda()
    tdt = torch.float16 if half else torch.float32
    tol = TOL_F16 if half else TOL_F32
    y = layer.forward(L.DeviceMatrix.from_numpy(x, dtype=tdt, ldim=h + pad)).to_numpy()
    mv = layer.m_mean_and_var.to_numpy()
    dx = layer.backward(L.DeviceMatrix.from_numpy(dy, dtype=tdt, ldim=h + pad)).to_numpy()
    mvg = layer.m_mean_and_var_gradient.to_numpy()
    out = dict(y=y, dx=dx, dscale=layer.m_scale_gradient.to_numpy(), dbias=layer.m_bias_gradient.to_numpy(),
               dmean=mvg[:, 0], dvar=mvg[:, 1], rmean=layer.weights[2].to_numpy(), rvar=layer.weights[3].to_numpy())
    if training:
        out.update(mean=mv[:, 0], var=mv[:, 1])
    ref, ex = {}, {}
    for dst, conv in ((ref, f32), (ex, f64)):
        xx, gg, sc, bi = conv(x), conv(dy), conv(scale), conv(bias)
        rm, rv = conv(rm0).copy(), conv(rv0).copy()
        dst["y"], dst["mean"], dst["var"] = orc.batch_norm_fwd(xx, C, cs, 1e-5, 0.9, sc, bi, rm, rv, bessel, training)
        dst["rmean"], dst["rvar"] = rm, rv
        dst["dx"], dst["dscale"], dst["dbias"], dst["dmean"], dst["dvar"] = orc.batch_norm_bwd(
            xx, gg, C, cs, 1e-5, dst["mean"], dst["var"], sc, rm, rv, bessel, training)
    return {k: check(f"batch_norm {k} dims={dims} w={w} half={half}", out[k], ref[k], ex[k], tol=tol) for k in out}


@pytest.mark.parametrize("w", [127, 128, 512, 513, 1024, 1025, 2048, 2049])
@pytest.mark.parametrize("half", [False, True])
def test_batch_norm_channel_per_workgroup_boundaries(L, w, half):
    """256 channels of 4 x 4 (fp16: 8 x 4) entries: the mini-batch sizes either side of every switch
    between 256, 512 and 1024 threads per channel, and between one workgroup per channel and the
    paths around it (fewer than 512 vectors, more than 8192; fp16 backward more than 4096)."""
    dims = (256, 8, 4) if half else (256, 4, 4)
    rng = np.random.default_rng(900 + w)
    h = int(np.prod(dims))
    x, dy = rand(rng, h, w, 2.0, 3.0), rand(rng, h, w)
    if half:
        x, dy = x.astype(np.float16).astype(np.float32), dy.astype(np.float16).astype(np.float32)
    scale = rng.uniform(0.5, 1.5, dims[0]).astype(np.float32)
    bias = (0.1 * rng.standard_normal(dims[0])).astype(np.float32)
    _bn_run(L, x, dy, dims, bool(w % 2), 0, scale, bias, half=half)


@pytest.mark.parametrize("dims,w,bessel,pad", BN_CASES)
def test_batch_norm(L, dims, w, bessel, pad):
    rng = np.random.default_rng(int(np.prod(dims)) + w)
    h = int(np.prod(dims))
    x, dy = rand(rng, h, w, 2.0, 3.0), rand(rng, h, w)
    C = dims[0]
    scale = rng.uniform(0.5, 1.5, C).astype(np.float32)
    bias = (0.1 * rng.standard_normal(C)).astype(np.float32)
    _bn_run(L, x, dy, dims, bessel, pad, scale, bias)


@pytest.mark.parametrize("dims,w,bessel,pad,training", [
    ((8, 16, 16), 12, True, 0, True), ((16, 28, 28), 8, False, 0, True), ((7, 5, 3), 14, True, 0, True),
    ((5, 24), 10, True, 8, True), ((256, 8, 8), 32, True, 0, True), ((3, 56, 56), 16, True, 0, False),
    ((2, 100000), 3, True, 0, True), ((64, 56, 56), 16, True, 0, True),
    # channels of whole fours but not eights, or a leading dimension padded by four: 8-byte accesses
    ((1024, 14, 14), 32, True, 0, True), ((256, 14, 14), 600, False, 0, True), ((6, 10, 10), 9, True, 0, False),
    ((16, 28, 28), 8, True, 4, True), ((40, 12), 64, True, 0, True), ((3, 4), 5, True, 4, True),
    # channels of odd sizes on matrices whose rows come in aligned fours: the row-tile kernels on fp16
    ((2048, 7, 7), 16, True, 0, True), ((4096,), 64, True, 0, True), ((64, 7, 7), 300, False, 0, True),
    ((12, 3, 3), 20, True, 0, True), ((1024, 1), 2048, True, 0, True), ((128, 7, 7), 10, True, 0, False),
    ((32, 7, 7), 64, True, 4, True), ((2000, 2), 200, False, 0, True), ((100, 12), 64, True, 0, True),
    ((8, 55, 55), 300, True, 0, True), ((4, 111, 111), 20, False, 0, True),
    # many channels of 512 to 8192 vectors: one workgroup keeps a channel (backward up to 4096 vectors of eight)
    ((512, 16, 16), 100, True, 0, True), ((300, 28, 28), 64, False, 0, True), ((1024, 14, 14), 128, True, 0, True),
    ((1100, 8), 600, True, 0, True),
    # odd maps, many channels: single halves in one workgroup's registers
    ((512, 7, 7), 100, True, 0, True), ((1024, 7, 7), 32, False, 0, True), ((300, 5, 5), 100, True, 0, True),
    ((256, 3, 3), 200, True, 1, True), ((130, 7, 7), 300, True, 0, True),
    ((3, 56, 56), 512, True, 0, True), ((2, 2000000), 1, True, 0, True),   # clusters of more than 64 workgroups
    ((3, 112, 112), 512, True, 0, True), ((2, 2500000), 2, False, 0, True)])   # streaming clusters
def test_batch_norm_f16(L, dims, w, bessel, pad, training):
    """fp16 storage, fp32 arithmetic: the oracle sees the fp16-rounded inputs."""
    rng = np.random.default_rng(int(np.prod(dims)) * 5 + w)
    h = int(np.prod(dims))
    x = rand(rng, h, w, 2.0, 3.0).astype(np.float16).astype(np.float32)
    dy = rand(rng, h, w).astype(np.float16).astype(np.float32)
    C = dims[0]
    scale = rng.uniform(0.5, 1.5, C).astype(np.float32)
    bias = (0.1 * rng.standard_normal(C)).astype(np.float32)
    _bn_run(L, x, dy, dims, bessel, pad, scale, bias, training=training, half=True)


def test_batch_norm_inference_and_reference_formula(L):
    rng = np.random.default_rng(77)
    dims, w = (6, 10, 10), 9
    h = int(np.prod(dims))
    x, dy = rand(rng, h, w, 2.0, 3.0), rand(rng, h, w)
    x[:100, :] = 4.0    # constant channel: variance is lifted to epsilon
    scale = rng.uniform(0.5, 1.5, 6).astype(np.float32)
    bias = (0.1 * rng.standard_normal(6)).astype(np.float32)
    _bn_run(L, x, dy, dims, True, 0, scale, bias, training=False)
    _bn_run(L, x, dy, dims, True, 0, scale, bias, mode=L.LBN_STATS_SUMSQ)
    _bn_run(L, x, dy, dims, True, 0, scale, bias)
    # the same three modes through the row-tile kernels (7 x 7 channels)
    dims, w = (16, 7, 7), 12
    h = int(np.prod(dims))
    x, dy = rand(rng, h, w, 2.0, 3.0), rand(rng, h, w)
    x[:49, :] = 4.0
    scale = rng.uniform(0.5, 1.5, 16).astype(np.float32)
    bias = (0.1 * rng.standard_normal(16)).astype(np.float32)
    _bn_run(L, x, dy, dims, True, 0, scale, bias, training=False)
    _bn_run(L, x, dy, dims, True, 0, scale, bias, mode=L.LBN_STATS_SUMSQ)
    _bn_run(L, x, dy, dims, False, 0, scale, bias)


def test_batch_norm_split_entry_points(L):
    """sums -> stats -> apply (the cut where a caller all-reduces) equals the fused call."""
    from lbann_amd import capi
    rng = np.random.default_rng(78)
    C, cs, w = 12, 64, 10
    h = C * cs
    x, dy = rand(rng, h, w, 2.0, 3.0), rand(rng, h, w)
    scale = rng.uniform(0.5, 1.5, C).astype(np.float32)
    bias = (0.1 * rng.standard_normal(C)).astype(np.float32)
    xm, gm = L.DeviceMatrix.from_numpy(x), L.DeviceMatrix.from_numpy(dy)
    ym, dm = L.DeviceMatrix(h, w), L.DeviceMatrix(h, w)
    dev = lambda a: torch.from_numpy(np.asarray(a, np.float32)).cuda()
    p = lambda t: capi.vp(t.data_ptr())
    mean, var, rm, rv = torch.empty(C).cuda(), torch.empty(C).cuda(), torch.zeros(C).cuda(), torch.ones(C).cuda()
    sc, bi = dev(scale), dev(bias)
    nb = capi.lib().lbn_batch_norm_workspace_bytes(C, cs, w)
    ws = torch.empty(max(nb, 1), dtype=torch.uint8, device="cuda")
    st = capi.vp(torch.cuda.current_stream().cuda_stream)
    capi.call("lbn_batch_norm_fwd_sums_f32", st, C, cs, w, xm.Buffer(), xm.ldim, p(mean), p(var), p(ws), nb)
    sums = mean.cpu().numpy().copy()
    assert rel_err(sums, x.astype(np.float64).reshape(cs, C, w, order="F").sum(axis=(0, 2))) < 1e-5
    capi.call("lbn_batch_norm_fwd_stats_f32", st, C, cs * w, 1, 1e-5, 0.9, p(mean), p(var), p(rm), p(rv))
    capi.call("lbn_batch_norm_fwd_apply_f32", st, C, cs, w, 1e-5, xm.Buffer(), xm.ldim, ym.Buffer(), ym.ldim,
              p(mean), p(var), p(sc), p(bi))
    rm0, rv0 = np.zeros(C, np.float32), np.ones(C, np.float32)
    y_ref, mean_ref, var_ref = orc.batch_norm_fwd(x, C, cs, 1e-5, 0.9, scale, bias, rm0, rv0)
    check("split y", ym.to_numpy(), y_ref, None)
    check("split mean", mean.cpu().numpy(), mean_ref, None)
    check("split var", var.cpu().numpy(), var_ref, None)
    check("split rmean", rm.cpu().numpy(), rm0, None)
    check("split rvar", rv.cpu().numpy(), rv0, None)
    ds, db, dmn, dvr = (torch.empty(C).cuda() for _ in range(4))
    capi.call("lbn_batch_norm_bwd_sums_f32", st, C, cs, w, 1e-5, xm.Buffer(), xm.ldim, gm.Buffer(), gm.ldim,
              p(mean), p(var), p(sc), p(ds), p(db), p(dmn), p(dvr), p(ws), nb)
    capi.call("lbn_batch_norm_bwd_apply_f32", st, C, cs, w, cs * w, 1, 1e-5, xm.Buffer(), xm.ldim, gm.Buffer(),
              gm.ldim, dm.Buffer(), dm.ldim, p(mean), p(var), p(sc), p(dmn), p(dvr))
    dx_ref, dg_ref, db_ref, dm_ref, dv_ref = orc.batch_norm_bwd(x, dy, C, cs, 1e-5, mean_ref, var_ref, scale)
    ex = orc.batch_norm_bwd(f64(x), f64(dy), C, cs, 1e-5, f64(mean_ref), f64(var_ref), f64(scale))
    check("split dx", dm.to_numpy(), dx_ref, ex[0])
    check("split dscale", ds.cpu().numpy(), dg_ref, ex[1])
    check("split dbias", db.cpu().numpy(), db_ref, ex[2])
    check("split dmean", dmn.cpu().numpy(), dm_ref, ex[3])
    check("split dvar", dvr.cpu().numpy(), dv_ref, ex[4])


# ===================================================================== golden fixtures on the GPU
def test_reference_fixtures_on_gpu(L, golden):
    F32_EPS = np.finfo(np.float32).eps
    met = lambda y: float(np.mean(np.sum(np.asarray(y, np.float64) ** 2, axis=0)))
    T = lambda a: np.asfortranarray(np.asarray(a).T)
    y = L.layer_norm_layer((31,)).forward(L.DeviceMatrix.from_numpy(T(golden["ln_x"]))).to_numpy()
    assert abs(met(y) - float(golden["ln_metric"])) <= 8 * float(golden["ln_metric"]) * F32_EPS
    assert rel_err(y.T, golden["ln_y"]) < TOL_F32
    ln = L.layer_norm_layer((31,), scale=True, bias=True, scale_values=golden["lna_scale"], bias_values=golden["lna_bias"])
    y = ln.forward(L.DeviceMatrix.from_numpy(T(golden["lna_x"]))).to_numpy()
    assert np.mean((y.T - golden["lna_y_test_scaled_bias"]) ** 2) <= 1e-8
    assert rel_err(y.T, golden["lna_y_exact"]) < TOL_F32
    for sd in (-1, 1, 0):
        y = L.layer_norm_layer((31, 2, 5), start_dim=sd).forward(
            L.DeviceMatrix.from_numpy(T(golden["lnm_x"].reshape(31, -1)))).to_numpy()
        assert np.mean((y.T - golden[f"lnm_y_test_sd{sd}"].reshape(31, -1)) ** 2) <= 1e-7
        assert rel_err(y.T, golden[f"lnm_y_exact_sd{sd}"].reshape(31, -1)) < TOL_F32
    for tag, rows in (("mb14", 14), ("all29", 29)):
        for bessel in (0, 1):
            bn = L.batch_normalization_layer((7, 5, 3), bessel_correction=bool(bessel))
            y = bn.forward(L.DeviceMatrix.from_numpy(T(golden["bn_x"][:rows]))).to_numpy()
            assert rel_err(y.T, golden[f"bn_{tag}_b{bessel}_y"]) < TOL_F32
            mv = bn.m_mean_and_var.to_numpy()
            assert rel_err(mv[:, 0], golden[f"bn_{tag}_b{bessel}_mean"]) < TOL_F32
            assert rel_err(mv[:, 1], golden[f"bn_{tag}_b{bessel}_var"]) < TOL_F32
    y = L.softmax_layer().forward(L.DeviceMatrix.from_numpy(T(golden["sm_x"]))).to_numpy()
    assert abs(met(y) - float(golden["sm_metric"])) <= 8 * float(golden["sm_metric"]) * F32_EPS
    assert rel_err(y.T, golden["sm_y"]) < TOL_F32
    y = L.log_softmax_layer().forward(L.DeviceMatrix.from_numpy(T(golden["lsm_x"]))).to_numpy()
    assert abs(met(y) - float(golden["lsm_metric"])) <= 8 * float(golden["lsm_metric"]) * F32_EPS
    assert rel_err(y.T, golden["lsm_y"]) < TOL_F32
    for tag, kw in (("default", {}), ("lastdim", dict(dim=-1, single_dim_mode=True))):
        y = L.channelwise_softmax_layer((5, 2, 7), **kw).forward(L.DeviceMatrix.from_numpy(T(golden["cws_x"]))).to_numpy()
        assert abs(met(y) - float(golden[f"cws_metric_{tag}"])) <= 8 * float(golden[f"cws_metric_{tag}"]) * F32_EPS
        assert rel_err(y.T, golden[f"cws_y_{tag}"]) < TOL_F32
    for tag, rows in (("mb14", 14), ("all29", 29)):
        eb = L.entrywise_batch_normalization_layer((7, 5, 3))
        y = eb.forward(L.DeviceMatrix.from_numpy(T(golden["ebn_x"][:rows]))).to_numpy()
        assert rel_err(y.T, golden[f"ebn_{tag}_y"]) < TOL_F32
        st = eb.m_batch_statistics.to_numpy()
        assert rel_err(st[:, 0], golden[f"ebn_{tag}_mean"]) < TOL_F32
        assert rel_err(st[:, 1], golden[f"ebn_{tag}_var"]) < TOL_F32
    y = L.instance_norm_layer((5, 3, 7)).forward(L.DeviceMatrix.from_numpy(T(golden["in_x"]))).to_numpy()
    assert abs(met(y) - float(golden["in_metric"])) <= 8 * float(golden["in_metric"]) * F32_EPS
    assert rel_err(y.T, golden["in_y"]) < TOL_F32


# ===================================================================== boundary behaviour
def test_empty_and_rejected_arguments(L):
    from lbann_amd import capi
    st = capi.vp(torch.cuda.current_stream().cuda_stream)
    null = capi.vp(None)
    lib = capi.lib()
    buf = torch.zeros(64, device="cuda")
    p = capi.vp(buf.data_ptr())
    # empty inputs: success, nothing launched, no pointer touched
    assert lib.lbn_softmax_fwd_f32(st, 0, 5, null, 0, null, 0, null, 0) == 0
    assert lib.lbn_softmax_fwd_f32(st, 8, 0, null, 8, null, 8, null, 0) == 0
    assert lib.lbn_layer_norm_fwd_f32(st, 1, 8, 8, 0, 1e-5, null, 8, null, 8, null, 2, null, null, null, 0, 0) == 0
    assert lib.lbn_batch_norm_fwd_f32(st, 0, 4, 4, 1, 1e-5, 0.9, 1, null, 0, null, 0, null, null, null, null, null, null, null, 0, 0) == 0
    assert lib.lbn_channelwise_softmax_bwd_f32(st, 4, 0, 0, 3, null, 0, null, 0, null, 0, null, 0) == 0
    # rejected arguments come back as negative status codes, never as a fault
    assert lib.lbn_softmax_fwd_f32(st, -1, 5, p, 8, p, 8, null, 0) == capi.LBN_ERR_INVALID_ARGUMENT
    assert lib.lbn_softmax_fwd_f32(st, 8, 2, p, 4, p, 8, null, 0) == capi.LBN_ERR_INVALID_ARGUMENT   # ld < height
    assert lib.lbn_softmax_fwd_f32(st, 8, 2, null, 8, p, 8, null, 0) == capi.LBN_ERR_INVALID_ARGUMENT
    assert lib.lbn_softmax_fwd_f32(st, 40001, 2, p, 40001, p, 40001, null, 0) == capi.LBN_ERR_WORKSPACE  # split path needs scratch
    assert lib.lbn_batch_norm_fwd_f32(st, 2, 4, 2, 1, 1e-5, 0.9, 1, p, 8, p, 8, p, p, p, p, p, p, null, 0, 0) == capi.LBN_ERR_WORKSPACE
    assert lib.lbn_layer_norm_bwd_f32(st, 1, 8, 8, 2, 1e-5, p, 8, p, 8, p, 8, p, 2, p, 2, null, p, null, null, 0) == capi.LBN_ERR_INVALID_ARGUMENT
    assert b"workspace" in lib.lbn_status_string(capi.LBN_ERR_WORKSPACE)
    with pytest.raises(L.LbnError):
        capi.call("lbn_softmax_fwd_f32", st, -1, 5, p, 8, p, 8, null, 0)
    with pytest.raises(ValueError):
        L.softmax_layer(mode="channel")
    with pytest.raises(ValueError):
        L.layer_norm_layer((4, 4), start_dim=2)
    torch.cuda.synchronize()


def test_results_are_bitwise_reproducible(L):
    """No atomics anywhere: two runs give identical bits (also a cheap race detector)."""
    rng = np.random.default_rng(99)
    x, dy = rand(rng, 4096, 300), rand(rng, 4096, 300)
    scale = (1 + 0.1 * rng.standard_normal(4096)).astype(np.float32)
    outs = []
    for _ in range(2):
        ln = L.layer_norm_layer((4096,), scale=True, bias=True, scale_values=scale, bias_values=scale)
        ln.forward(L.DeviceMatrix.from_numpy(x))
        ln.backward(L.DeviceMatrix.from_numpy(dy))
        bn = L.batch_normalization_layer((16, 256))
        yb = bn.forward(L.DeviceMatrix.from_numpy(x)).to_numpy()
        db = bn.backward(L.DeviceMatrix.from_numpy(dy)).to_numpy()
        outs.append([ln.error_signals.to_numpy(), ln.m_scale_gradient.to_numpy(), ln.m_bias_gradient.to_numpy(),
                     yb, db, bn.m_scale_gradient.to_numpy()])
    for a, b in zip(*outs):
        assert np.array_equal(a, b)


def test_rendezvous_flag_stays_clear(L):
    """The kernels in which workgroups wait for each other (batch norm channels, softmax rows
    shared by a cluster) leave the time-out flag of their workspace clear."""
    import ctypes
    from lbann_amd import capi
    rng = np.random.default_rng(77)
    flag = ctypes.c_int(-1)
    stream = capi.vp(torch.cuda.current_stream().cuda_stream)
    bn = L.batch_normalization_layer((16, 28, 28))
    bn.forward(L.DeviceMatrix.from_numpy(rand(rng, 16 * 784, 8)))
    bn.backward(L.DeviceMatrix.from_numpy(rand(rng, 16 * 784, 8)))
    capi.call("lbn_workspace_timed_out", stream, capi.vp(bn._ws.buf.data_ptr()), ctypes.byref(flag))
    assert flag.value == 0
    sm = L.softmax_layer()
    sm.forward(L.DeviceMatrix.from_numpy(rand(rng, 262148, 48)))   # rows shared by clusters
    flag.value = -1
    capi.call("lbn_workspace_timed_out", stream, capi.vp(sm._ws.buf.data_ptr()), ctypes.byref(flag))
    assert flag.value == 0
    capi.call("lbn_workspace_timed_out", stream, capi.vp(None), ctypes.byref(flag))
    assert flag.value == 0


def test_concurrent_host_threads_on_separate_streams(L):
    """Two host threads drive different layers on their own streams at the same time (the
    entry points are re-entrant: per-call tags, a locked occupancy cache, caller-owned
    scratch); each result equals the one the same call gives on its own."""
    import threading
    rng = np.random.default_rng(91)
    xs, xb = rand(rng, 262148, 48), rand(rng, 16 * 784, 32, 2.0, 3.0)   # row clusters / channel clusters
    xl = rand(rng, 4096, 300)

    def run_softmax(out):
        s = torch.cuda.Stream()
        with torch.cuda.stream(s):
            out.append([L.softmax_layer().forward(L.DeviceMatrix.from_numpy(xs)).to_numpy() for _ in range(4)])

    def run_norms(out):
        s = torch.cuda.Stream()
        with torch.cuda.stream(s):
            r = []
            for _ in range(4):
                r.append(L.batch_normalization_layer((16, 28, 28)).forward(L.DeviceMatrix.from_numpy(xb)).to_numpy())
                r.append(L.layer_norm_layer((4096,)).forward(L.DeviceMatrix.from_numpy(xl)).to_numpy())
            out.append(r)

    alone_a, alone_b = [], []
    run_softmax(alone_a)
    run_norms(alone_b)
    got_a, got_b = [], []
    ta, tb = threading.Thread(target=run_softmax, args=(got_a,)), threading.Thread(target=run_norms, args=(got_b,))
    ta.start(); tb.start(); ta.join(); tb.join()
    torch.cuda.synchronize()
    for a, b in zip(alone_a[0] + alone_b[0], got_a[0] + got_b[0]):
        assert np.array_equal(a, b)


def test_cluster_kernels_enqueued_on_two_streams_without_waiting(L):
    """Kernels whose workgroups wait for each other must not share the device.  One host thread
    enqueues many of them on two streams, alternately and without waiting in between: the library
    orders them across the streams itself, every result equals the one computed on one stream, and
    no wait runs out (to_numpy() checks the workspaces' error words)."""
    rng = np.random.default_rng(17)
    xs = rand(rng, 262144, 8)                     # a few long rows: row clusters
    xb = rand(rng, 64 * 784, 64, 2.0, 3.0)        # channel clusters
    sm_ref = L.softmax_layer().forward(L.DeviceMatrix.from_numpy(xs)).to_numpy()
    bn_ref = L.batch_normalization_layer((64, 28, 28)).forward(L.DeviceMatrix.from_numpy(xb)).to_numpy()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    reps = 12
    sms = [L.softmax_layer() for _ in range(reps)]
    bns = [L.batch_normalization_layer((64, 28, 28)) for _ in range(reps)]
    dxs, dxb = L.DeviceMatrix.from_numpy(xs), L.DeviceMatrix.from_numpy(xb)
    torch.cuda.synchronize()
    ys, yb = [], []
    for i in range(reps):
        with torch.cuda.stream(s1):
            ys.append(sms[i].forward(dxs))
        with torch.cuda.stream(s2):
            yb.append(bns[i].forward(dxb))
    torch.cuda.synchronize()
    for y in ys:
        assert np.array_equal(y.to_numpy(), sm_ref)
    for y in yb:
        assert np.array_equal(y.to_numpy(), bn_ref)



def test_cluster_kernels_from_two_host_threads_on_the_per_thread_stream(L, monkeypatch):
    """hipStreamPerThread is one handle that names a different stream in every host thread, so two
    threads that pass it enqueue on two streams: the library must still keep their cluster kernels
    apart.  Every result equals the one computed alone and no wait runs out."""
    import threading

    from lbann_amd import capi

    rng = np.random.default_rng(23)
    xs = rand(rng, 262144, 8)                     # a few long rows: row clusters
    xb = rand(rng, 64 * 784, 64, 2.0, 3.0)        # channel clusters
    sm_ref = L.softmax_layer().forward(L.DeviceMatrix.from_numpy(xs)).to_numpy()
    bn_ref = L.batch_normalization_layer((64, 28, 28)).forward(L.DeviceMatrix.from_numpy(xb)).to_numpy()
    dxs, dxb = L.DeviceMatrix.from_numpy(xs), L.DeviceMatrix.from_numpy(xb)
    reps = 12
    sms = [L.softmax_layer() for _ in range(reps)]
    bns = [L.batch_normalization_layer((64, 28, 28)) for _ in range(reps)]
    # first calls on the ordinary stream: the workspaces are allocated outside the threads
    ys = [m.forward(dxs) for m in sms]
    yb = [m.forward(dxb) for m in bns]
    torch.cuda.synchronize()
    ys, yb = [None] * reps, [None] * reps
    monkeypatch.setattr(L, "_stream", lambda: capi.vp(2))  # hipStreamPerThread
    errors = []

    def run(layers, x, out):
        try:
            torch.cuda.set_device(0)
            for i, m in enumerate(layers):
                out[i] = m.forward(x)
        except Exception as e:  # surfaced below: an exception in a thread would otherwise be lost
            errors.append(e)

    ta = threading.Thread(target=run, args=(sms, dxs, ys))
    tb = threading.Thread(target=run, args=(bns, dxb, yb))
    ta.start(); tb.start(); ta.join(); tb.join()
    torch.cuda.synchronize()
    monkeypatch.undo()
    assert not errors, errors
    for y in ys:
        assert np.array_equal(y.to_numpy(), sm_ref)
    for y in yb:
        assert np.array_equal(y.to_numpy(), bn_ref)


# ---------------------------------------------------------------- the reference's summation order
def _bits_equal(name, a, b):
    a, b = np.ascontiguousarray(a, np.float32), np.ascontiguousarray(b, np.float32)
    assert a.shape == b.shape and a.tobytes() == b.tobytes(), \
        f"{name}: not bit-equal to the fp32 reference (max abs difference {np.abs(a - b).max():.3e})"


@pytest.mark.parametrize("dims,w,bessel,pad,half", [
    ((8, 16, 16), 12, True, 0, False), ((7, 5, 3), 14, False, 0, False), ((5, 24), 10, True, 8, False),
    ((3, 1001), 7, True, 3, False), ((4, 1), 1, True, 0, False), ((6, 1), 33, True, 0, False),
    ((16, 14, 14), 9, True, 0, True), ((5, 7, 7), 20, False, 1, True)])
def test_batch_norm_reference_order_is_bit_equal(L, dims, w, bessel, pad, half):
    """LBN_STATS_REFERENCE_ORDER: statistics and the four per-channel gradients equal the
    restated CPU code's bit for bit (any alignment, channel size, fp16 storage; a channel of
    one entry in all keeps the reference's special case)."""
    rng = np.random.default_rng(int(np.prod(dims)) * 31 + w)
    h = int(np.prod(dims))
    x, dy = rand(rng, h, w, 2.0, 3.0), rand(rng, h, w)
    if half:
        x, dy = f32(x.astype(np.float16)), f32(dy.astype(np.float16))
    C = dims[0]
    scale = rng.uniform(0.5, 1.5, C).astype(np.float32)
    bias = (0.1 * rng.standard_normal(C)).astype(np.float32)
    cs = h // C
    layer = L.batch_normalization_layer(dims, 0.9, 1e-5, bessel, scale, bias, stats_mode=L.LBN_STATS_REFERENCE_ORDER)
    tdt = torch.float16 if half else torch.float32
    y = layer.forward(L.DeviceMatrix.from_numpy(x, dtype=tdt, ldim=h + pad)).to_numpy()
    mv = layer.m_mean_and_var.to_numpy()
    rm, rv = np.zeros(C, np.float32), np.ones(C, np.float32)
    y_ref, m_ref, v_ref = orc.batch_norm_fwd(x, C, cs, 1e-5, 0.9, scale, bias, rm, rv, bessel)
    _bits_equal("mean", mv[:, 0], m_ref)
    _bits_equal("var", mv[:, 1], v_ref)
    _bits_equal("running mean", layer.weights[2].to_numpy(), rm)
    _bits_equal("running var", layer.weights[3].to_numpy(), rv)
    check(f"batch_norm reference-order y dims={dims}", y, y_ref, tol=TOL_F16 if half else TOL_F32)
    if half:
        return  # the backward of this mode is fp32 only
    dx = layer.backward(L.DeviceMatrix.from_numpy(dy, ldim=h + pad)).to_numpy()
    mvg = layer.m_mean_and_var_gradient.to_numpy()
    dx_ref, dg_ref, db_ref, dm_ref, dv_ref = orc.batch_norm_bwd(x, dy, C, cs, 1e-5, m_ref, v_ref, scale, bessel=bessel)
    _bits_equal("dscale", layer.m_scale_gradient.to_numpy(), dg_ref)
    _bits_equal("dbias", layer.m_bias_gradient.to_numpy(), db_ref)
    _bits_equal("dmean", mvg[:, 0], dm_ref)
    _bits_equal("dvar", mvg[:, 1], dv_ref)
    check(f"batch_norm reference-order dx dims={dims}", dx, dx_ref)


@pytest.mark.parametrize("dims,start_dim,w,affine,pad,half", [
    ((1024,), 0, 64, True, 0, False), ((31,), 0, 15, False, 0, False), ((8, 512), -1, 9, True, 5, False),
    ((1,), 0, 6, True, 0, False), ((3, 777), 1, 11, True, 1, False), ((2, 4096), 1, 33, True, 0, True),
    ((1001,), 0, 17, False, 3, True)])
def test_layer_norm_reference_order_is_bit_equal(L, dims, start_dim, w, affine, pad, half):
    """LBN_STATS_REFERENCE_ORDER: mean, variance and y equal the restated CPU code's bit for
    bit (fp16 storage: y equal after rounding to binary16); columns with |mean| >> stdev keep
    the reference's cancellation."""
    rng = np.random.default_rng(int(np.prod(dims)) * 17 + w)
    h = int(np.prod(dims))
    x = rand(rng, h, w, 0.3, 1.5)
    x[:, ::3] += 300.0   # E[x^2] - mean^2 cancels in fp32 here
    x = np.asfortranarray(x)
    if half:
        x = f32(x.astype(np.float16))
    n = int(np.prod(dims[(start_dim if start_dim >= 0 else len(dims) + start_dim):]))
    scale = (1 + 0.3 * rng.standard_normal(n)).astype(np.float32)
    bias = (0.3 * rng.standard_normal(n)).astype(np.float32)
    kw = dict(scale_values=scale, bias_values=bias) if affine else {}
    layer = L.layer_norm_layer(dims, 1e-5, affine, affine, start_dim, stats_mode=L.LBN_STATS_REFERENCE_ORDER, **kw)
    G = layer.num_normalized
    tdt = torch.float16 if half else torch.float32
    y = layer.forward(L.DeviceMatrix.from_numpy(x, dtype=tdt, ldim=h + pad)).to_numpy()
    y_ref, st_ref = orc.layer_norm_fwd(x, G, n, n, 1e-5, scale if affine else None, bias if affine else None)
    _bits_equal("statistics", layer.m_statistics.to_numpy(), st_ref)
    if half:
        _bits_equal("y", f32(y), f32(y_ref.astype(np.float16)))
    else:
        _bits_equal("y", y, y_ref)


# ===================================================================== diagnostics
@pytest.mark.parametrize("C,cs,w,pad", [(5, 12, 7, 4), (1, 4, 1, 0), (3, 100000, 2, 0), (40, 3136, 16, 0),
                                        (256, 3136, 64, 0), (700, 8, 300, 8), (2, 2048 * 4 * 3, 5, 0)])
@pytest.mark.parametrize("channel_major", [0, 1])
def test_selftest_copy_pipeline_copies_bit_for_bit(L, C, cs, w, pad, channel_major):
    """The copy that stands for the batch-norm cluster kernels' order of accesses moves every
    entry once and touches nothing else."""
    h = C * cs
    ld = h + pad
    x = L.DeviceMatrix(h, w, ldim=ld)
    x.tensor.normal_()
    y = L.DeviceMatrix(h, w, ldim=ld, fill=-7.0)
    L.call("lbn_selftest_copy_pipeline_f32", L._stream(), C, cs, w, x.Buffer(), x.ldim, y.Buffer(), y.ldim,
           channel_major)
    torch.cuda.synchronize()
    assert torch.equal(y.tensor[:, :h], x.tensor[:, :h])
    if pad:
        assert bool((y.tensor[:, h:] == -7.0).all())


def test_selftest_copy_pipeline_rejects_what_it_cannot_copy(L):
    x = L.DeviceMatrix(24, 3)
    y = L.DeviceMatrix(24, 3)
    lib = L.capi.lib()
    st = L._stream()
    assert lib.lbn_selftest_copy_pipeline_f32(st, 4, 6, 3, x.Buffer(), 24, y.Buffer(), 24, 1) == L.capi.LBN_ERR_UNSUPPORTED
    assert lib.lbn_selftest_copy_pipeline_f32(st, 2, 12, 3, x.Buffer(), 20, y.Buffer(), 24, 0) == L.capi.LBN_ERR_INVALID_ARGUMENT
    assert lib.lbn_selftest_copy_pipeline_f32(st, 2, 12, 3, None, 24, y.Buffer(), 24, 0) == L.capi.LBN_ERR_INVALID_ARGUMENT
    assert lib.lbn_selftest_copy_pipeline_f32(st, 0, 12, 3, None, 0, None, 0, 1) == L.capi.LBN_OK


@pytest.mark.parametrize("h,w,pad", [(105, 29, 0), (4096, 64, 4), (1000, 1, 0), (260, 300, 0), (100000, 33, 0),
                                     (7, 2, 1)])
def test_entrywise_batch_norm_reference_order_is_bit_equal(L, h, w, pad):
    """The test-only forward that adds in the CPU code's order and applies its unclamped variance
    gives the CPU code's bits: the default kernels differ from it by summation order and the clamp."""
    rng = np.random.default_rng(11 * h + w)
    x = rand(rng, h, w, 3.0, 0.5)   # |mean| >> sigma: E[x^2] - mean^2 cancels
    rm0 = rng.normal(size=h).astype(np.float32)
    rv0 = rng.uniform(0.5, 2.0, size=h).astype(np.float32)
    rm, rv = rm0.copy(), rv0.copy()
    y_ref, st_ref = orc.entrywise_batch_norm_fwd(f32(x), 0.9, 1e-5, rm, rv, True)
    xd = L.DeviceMatrix.from_numpy(x, ldim=h + pad)
    yd = L.DeviceMatrix(h, w, ldim=h + pad)
    st = L.DeviceMatrix(h, 2)
    rmd, rvd = L._Vector(h, "cuda", rm0), L._Vector(h, "cuda", rv0)
    L.call("lbn_entrywise_batch_norm_fwd_reference_order_f32", L._stream(), h, w, 0.9, 1e-5, xd.Buffer(), xd.ldim,
           yd.Buffer(), yd.ldim, st.Buffer(), st.ldim, rmd.Buffer(), rvd.Buffer())
    _bits_equal("entrywise_bn reference-order stats", st.to_numpy(), st_ref)
    _bits_equal("entrywise_bn reference-order y", yd.to_numpy(), y_ref)
    _bits_equal("entrywise_bn reference-order running mean", rmd.to_numpy(), rm)
    _bits_equal("entrywise_bn reference-order running var", rvd.to_numpy(), rv)


def test_entrywise_batch_norm_reference_order_keeps_the_negative_variance(L):
    """Where the default kernels clamp E[x^2] - mean^2 at zero, the reference-order forward returns what
    the CPU code returns: the negative variance and NaN outputs for that entry."""
    x = f32(np.array([[3198.374755859375, 3198.375], [1.0, 3.0], [0.5, -0.5], [2.0, 2.0]], dtype=np.float32))
    rm, rv = np.zeros(4, np.float32), np.ones(4, np.float32)
    y_ref, st_ref = orc.entrywise_batch_norm_fwd(f32(x), 0.9, 1e-5, rm, rv, True)
    assert st_ref[0, 1] < 0 and np.isnan(y_ref[0]).all()
    xd, yd, st = L.DeviceMatrix.from_numpy(x), L.DeviceMatrix(4, 2), L.DeviceMatrix(4, 2)
    rmd, rvd = L._Vector(4, "cuda", np.zeros(4)), L._Vector(4, "cuda", np.ones(4))
    L.call("lbn_entrywise_batch_norm_fwd_reference_order_f32", L._stream(), 4, 2, 0.9, 1e-5, xd.Buffer(), xd.ldim,
           yd.Buffer(), yd.ldim, st.Buffer(), st.ldim, rmd.Buffer(), rvd.Buffer())
    _bits_equal("stats", st.to_numpy(), st_ref)
    y = yd.to_numpy()
    assert np.isnan(y[0]).all()
    _bits_equal("y of the other entries", y[1:], y_ref[1:])
    _bits_equal("running var", rvd.to_numpy(), rv)
