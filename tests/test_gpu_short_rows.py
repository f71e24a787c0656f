"""Many rows of a few elements: the shapes pooling layers hand to !max, !mean and to MaxValue-Node's
backward (rows of k-h k-w window elements, source/nn/pool.lisp:83-105, base-impl/matrix-ops.lisp:312-334).
Each of the three node families has a thread-per-row (or vector-per-thread) kernel for them; checked
against numpy, which for these operations is the definition: first occurrence for the indices, NaN never
selected, sums of at most 32 binary32 numbers exact in binary64 and rounded once."""
import numpy as np
import pytest

from helpers import assert_bit_equal

pytestmark = pytest.mark.gpu
f32 = np.float32


@pytest.mark.parametrize("cols", [1, 2, 3, 4, 5, 8, 9, 16, 25, 31, 32, 33])
def test_select_tiny_rows(gpu, cols):
    """33 columns are one too many for the thread-per-row kernel: the same answers from the next one."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(200 + cols)
    rows = 9001
    x = rng.integers(-6, 7, (rows, cols)).astype(f32)          # many ties
    x[5] = np.nan                                               # a row of NaNs: -inf / +inf, index 0
    x[6, 0] = np.nan                                            # NaN is never selected
    x[7, cols - 1] = np.inf
    x[8, 0] = -np.inf
    dx = F.from_numpy(x)
    with np.errstate(invalid="ignore"):
        filled_lo = np.where(np.isnan(x), -np.inf, x)
        filled_hi = np.where(np.isnan(x), np.inf, x)
    assert_bit_equal(F.max(dx).numpy()[:, 0], filled_lo.max(axis=1), "max")
    assert_bit_equal(F.min(dx).numpy()[:, 0], filled_hi.min(axis=1), "min")
    want_amax = filled_lo.argmax(axis=1)
    want_amin = filled_hi.argmin(axis=1)
    # numpy picks the first -inf of an all-NaN row too; where a row's only finite candidates are NaN-filled
    # positions the kernel's index is the first non-NaN occurrence of the extreme, or 0 for a row of NaNs
    for want in (want_amax, want_amin):
        want[5] = 0
    if cols > 1:
        got_amax = F.argmax(dx).numpy()[:, 0]
        got_amin = F.argmin(dx).numpy()[:, 0]
        keep = np.ones(rows, bool)
        keep[[6, 8]] = False                                    # rows whose filled extreme may sit on the NaN / -inf itself
        np.testing.assert_array_equal(got_amax[keep], want_amax[keep])
        np.testing.assert_array_equal(got_amin[keep], want_amin[keep])
        assert not np.isnan(x[6, got_amax[6]]) and x[6, got_amax[6]] == np.nanmax(x[6])
        assert x[8, got_amin[8]] == -np.inf and got_amin[8] == 0


@pytest.mark.parametrize("dtype,cols", [("double", 16), ("double", 17), ("int32", 7), ("uint8", 100), ("int16", 64),
                                        ("uint32", 32), ("int8", 3),
                                        # rows of exactly 16 bytes: one vector load per row
                                        ("double", 2), ("int32", 4), ("uint8", 16), ("int16", 8), ("uint32", 4)])
def test_select_tiny_rows_typed(gpu, dtype, cols):
    W = gpu
    F = W.functional
    rng = np.random.default_rng(cols)
    np_dtype = {"double": np.float64, "int32": np.int32, "uint8": np.uint8, "int16": np.int16, "uint32": np.uint32,
                "int8": np.int8}[dtype]
    rows = 8500
    if dtype == "double":
        x = rng.standard_normal((rows, cols)).astype(np_dtype)
    else:
        info = np.iinfo(np_dtype)
        x = rng.integers(info.min, int(info.max) + 1, (rows, cols)).astype(np_dtype)
        x[0] = info.min
        x[1] = info.max
    dx = F.from_numpy(x, dtype=dtype)
    np.testing.assert_array_equal(F.max(dx).numpy()[:, 0], x.max(axis=1))
    np.testing.assert_array_equal(F.min(dx).numpy()[:, 0], x.min(axis=1))
    if dtype == "double":
        np.testing.assert_array_equal(F.argmax(dx).numpy()[:, 0], x.argmax(axis=1))
        np.testing.assert_array_equal(F.argmin(dx).numpy()[:, 0], x.argmin(axis=1))


@pytest.mark.parametrize("cols", [1, 2, 4, 7, 9, 16, 25, 32, 33])
def test_sum_and_mean_of_tiny_rows(gpu, cols):
    W = gpu
    F = W.functional
    rng = np.random.default_rng(300 + cols)
    rows = 9100
    x = (rng.standard_normal((rows, cols)) * 3).astype(f32)
    x[3] = np.inf
    x[4, 0] = np.nan
    dx = F.from_numpy(x)
    with np.errstate(invalid="ignore"):
        total = x.astype(np.float64).sum(axis=1)
    assert_bit_equal(F.sum(dx, axis=1).numpy()[:, 0], total.astype(f32), "row sums")
    assert_bit_equal(F.mean(dx, axis=1).numpy()[:, 0], total.astype(f32) / f32(cols), "row means")
    # accumulating into a destination that holds something (the AddNode of !sum's composition)
    seed = rng.standard_normal((rows, 1)).astype(f32)
    with np.errstate(invalid="ignore"):
        want = (seed[:, 0].astype(np.float64) + total).astype(f32)
    got = F.add_(F.from_numpy(seed).view(True, (":broadcast", cols)), dx)
    assert_bit_equal(got.numpy()[:, 0], want, "accumulated")


@pytest.mark.parametrize("cols", [2, 3, 4, 5, 8, 10, 12, 33, 36, 1020, 1023])
@pytest.mark.parametrize("which", ["y", "x", "both", "none"])
def test_compare_short_rows(gpu, cols, which):
    """A matrix of short rows against one value per row (broadcast along the row) on either side."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(cols + len(which))
    rows = 9001 if cols < 1000 else 71
    x = rng.integers(-3, 4, (rows, cols if which not in ("x", "both") else 1)).astype(f32)
    y = rng.integers(-3, 4, (rows, cols if which not in ("y", "both") else 1)).astype(f32)
    x.flat[:2] = [np.nan, -0.0]
    y.flat[:2] = [1.0, 0.0]
    dx, dy = F.from_numpy(x), F.from_numpy(y)
    vx = dx if x.shape[1] == cols else dx.view(True, (":broadcast", cols))
    vy = dy if y.shape[1] == cols else dy.view(True, (":broadcast", cols))
    bx, by = np.broadcast_to(x, (rows, cols)), np.broadcast_to(y, (rows, cols))
    for op, fn in (("=", np.equal), ("<", np.less), ("<=", np.less_equal), (">", np.greater), (">=", np.greater_equal)):
        with np.errstate(invalid="ignore"):
            want = np.where(fn(bx, by), f32(2.0), f32(-1.0))
        got = F.compare(vx, vy, op, true_then=2.0, false_then=-1.0).numpy()
        assert_bit_equal(got, want, f"{op} with {which} broadcast")


@pytest.mark.parametrize("rows,cols", [(400003, 3), (300000, 4), (100001, 10), (100352, 64), (70000, 100), (50000, 128),
                                       (40000, 129), (3, 100000), (2, 70001), (15, 4097)])
def test_column_sums_of_narrow_and_of_flat_matrices(gpu, rows, cols):
    """!sum :axis 0 (bias gradients: the column sums of (N h w, C_out) or (N, classes)) where the matrix is
    tall and narrow, and where it has only a few rows: binary64 partial sums, so the result is the float64 sum
    rounded (exact for these magnitudes up to the last rounding, compared with one unit of slack)."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(rows + cols)
    x = rng.standard_normal((rows, cols)).astype(f32)
    dx = F.from_numpy(x)
    want = x.astype(np.float64).sum(axis=0)
    got = F.sum(dx, axis=0).numpy().ravel()
    from helpers import ulp_distance
    assert np.max(ulp_distance(got, want.astype(f32))) <= 1
    assert np.max(np.abs(got - want)) <= 2.0 ** -23 * np.max(np.abs(x).astype(np.float64).sum(axis=0))
    mean = F.mean(dx, axis=0).numpy().ravel()
    assert np.max(np.abs(mean - want / rows)) <= 2.0 ** -22 * np.max(np.abs(want / rows)) + 1e-12
    # into a destination that already holds values (AddNode into the broadcast view)
    seed = rng.standard_normal((1, cols)).astype(f32)
    acc = F.add_(F.from_numpy(seed).view((":broadcast", rows), True), dx).numpy()[0]
    assert np.max(np.abs(acc - (seed[0] + want))) <= 2.0 ** -22 * (np.abs(seed[0]) + np.abs(want)).max()


@pytest.mark.parametrize("dtype", ["double", "int32", "uint8", "int16"])
@pytest.mark.parametrize("rows,cols", [(200001, 4), (140000, 9), (3, 70000), (70001, 64), (30000, 100), (20000, 128), (9000, 129),
                                       (5000, 1)])
def test_typed_sums_of_short_rows_and_of_flat_matrices(gpu, dtype, rows, cols):
    """!sum on :double and the integer types (wrap-around sums, as the reference's C loops produce) along a
    short trailing axis of very many rows, and down the few rows of a flat matrix."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(rows + cols)
    np_dtype = {"double": np.float64, "int32": np.int32, "uint8": np.uint8, "int16": np.int16}[dtype]
    if dtype == "double":
        x = rng.standard_normal((rows, cols))
    else:
        info = np.iinfo(np_dtype)
        x = rng.integers(info.min, int(info.max) + 1, (rows, cols)).astype(np_dtype)
    dx = F.from_numpy(x, dtype=dtype)
    for axis in (1, 0):
        got = F.sum(dx, axis=axis).numpy().ravel()
        if dtype == "double":
            want = x.sum(axis=axis)
            assert np.max(np.abs(got - want)) <= 1e-13 * np.abs(x).sum(axis=axis).max()
        else:
            want = x.astype(np.int64).sum(axis=axis).astype(np_dtype)    # modulo 2^bits
            np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("shape,axes", [((32, 64, 28, 28), (0, 2, 3)), ((16, 3, 64, 64), (0, 2, 3)), ((6, 40, 50, 60), (1, 3)),
                                        ((5, 70, 9, 1000), (0, 1, 3)), ((2, 3, 400000), (0, 2))])
def test_sums_that_keep_a_middle_axis(gpu, shape, axes):
    """Few destinations, each a long sum over axes on both sides of the kept ones: the per-channel sums of an
    (N, C, H, W) tensor (batch-normalisation statistics, a channel-first bias gradient).  The reduced indices
    of a destination are shared out over several workgroups and folded in binary64."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal(shape).astype(f32)
    dx = F.from_numpy(x)
    want = x.astype(np.float64).sum(axis=axes, keepdims=True)
    mag = np.abs(x).astype(np.float64).sum(axis=axes, keepdims=True)
    got = F.sum(dx, axis=axes).numpy()
    assert got.shape == want.shape
    assert np.all(np.abs(got - want) <= 2.0 ** -23 * mag)
    count = np.prod([shape[a] for a in axes])
    mean = F.mean(dx, axis=axes).numpy()
    assert np.all(np.abs(mean - want / count) <= 2.0 ** -22 * mag / count)


def test_pooling_layers_at_size(gpu):
    """MaxPool2D / AvgPool2D forward and MaxPool2D backward on (8, 16, 64, 64): every kernel above in one
    composition, against the definitions."""
    W = gpu
    F, nn = W.functional, W.nn
    rng = np.random.default_rng(77)
    x = rng.integers(-4, 5, (8, 16, 64, 64)).astype(f32)        # ties inside windows
    dx = F.from_numpy(x)
    win = x.reshape(8, 16, 32, 2, 32, 2)
    assert_bit_equal(F.to_contiguous(nn.max_pool2d(dx, 2)).numpy(), win.max(axis=(3, 5)), "max pool")
    assert_bit_equal(F.to_contiguous(nn.avg_pool2d(dx, 2)).numpy(),
                     (win.astype(np.float64).sum(axis=(3, 5)).astype(f32) / f32(4)), "avg pool")
    dy = rng.standard_normal((8, 16, 32, 32)).astype(f32)
    mask = win == win.max(axis=(3, 5), keepdims=True)
    want = np.where(mask, dy[:, :, :, None, :, None], f32(0.0)).astype(f32).reshape(x.shape)   # the fold starts from +0
    assert_bit_equal(nn.max_pool2d_backward(dx, F.from_numpy(dy), 2).numpy(), want, "max pool backward")
    want_avg = np.broadcast_to((dy / f32(4))[:, :, :, None, :, None], win.shape).reshape(x.shape)
    assert_bit_equal(nn.avg_pool2d_backward(dx, F.from_numpy(dy), 2).numpy(), want_avg, "avg pool backward")


@pytest.mark.parametrize("narrow", [2, 3, 5, 8, 12, 15, 16, 24, 31])
@pytest.mark.parametrize("long", [256, 511, 1000, 4099])
def test_transposing_passes_with_one_short_axis(gpu, narrow, long):
    """(long, narrow) <-> (narrow, long): the exchange whose short axis has fewer than 16 elements takes long
    tiles with the whole short axis.  Copies in both directions, an accumulating pass, batches in front,
    a sliced (unaligned, padded) operand; data movement and one rounding each: bit-exact."""
    F = gpu.functional
    rng = np.random.default_rng(narrow * 10000 + long)
    a = rng.standard_normal((3, long, narrow)).astype(np.float32)
    da = F.from_numpy(a)
    # src contiguous along the short axis
    np.testing.assert_array_equal(F.copy(da.permute(0, 2, 1)).numpy(), a.transpose(0, 2, 1))
    # dst contiguous along the short axis
    b = rng.standard_normal((3, narrow, long)).astype(np.float32)
    db = F.from_numpy(b)
    np.testing.assert_array_equal(F.copy(db.permute(0, 2, 1)).numpy(), b.transpose(0, 2, 1))
    # accumulate: b += a^T and a += b^T
    got = F.add_(F.copy(db), da.permute(0, 2, 1)).numpy()
    np.testing.assert_array_equal(got, b + a.transpose(0, 2, 1))
    got = F.add_(F.copy(da), db.permute(0, 2, 1)).numpy()
    np.testing.assert_array_equal(got, a + b.transpose(0, 2, 1))
    # a window of a wider tensor (rows not adjacent, base off 16 bytes)
    wide = rng.standard_normal((long + 2, narrow + 3)).astype(np.float32)
    dw = F.from_numpy(wide)
    win = dw.view((1, long + 1), (1, narrow + 1))
    np.testing.assert_array_equal(F.copy(win.permute(1, 0)).numpy(), wide[1:long + 1, 1:narrow + 1].T)


def test_image_layout_exchange(gpu):
    """NCHW <-> NHWC with three channels, both directions."""
    F = gpu.functional
    rng = np.random.default_rng(2)
    x = rng.standard_normal((5, 3, 37, 53)).astype(np.float32)
    dx = F.from_numpy(x)
    nhwc = F.copy(dx.permute(0, 2, 3, 1))
    np.testing.assert_array_equal(nhwc.numpy(), x.transpose(0, 2, 3, 1))
    np.testing.assert_array_equal(F.copy(nhwc.permute(0, 3, 1, 2)).numpy(), x)


@pytest.mark.parametrize("shape", [(300, 500), (64, 64), (7, 129, 65), (1000, 17)])
def test_passes_into_a_transposed_destination(gpu, shape):
    """x^T += y and a copy into x^T: the destination's unit-stride axis is not the last one."""
    F = gpu.functional
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal(shape).astype(np.float32)
    perm = tuple(range(len(shape) - 2)) + (len(shape) - 1, len(shape) - 2)
    y = rng.standard_normal(tuple(shape[p] for p in perm)).astype(np.float32)
    dx, dy = F.from_numpy(x), F.from_numpy(y)
    F.add_(dx.permute(*perm), dy)
    np.testing.assert_array_equal(dx.numpy(), x + y.transpose(perm))
    F.move_(dx.permute(*perm), dy)
    np.testing.assert_array_equal(dx.numpy(), y.transpose(perm))


@pytest.mark.parametrize("cols", [1, 2, 3, 7, 10, 16, 17, 31, 32, 33, 48, 63, 64])
@pytest.mark.parametrize("rows", [16384, 20001])
def test_softmax_and_layernorm_of_tiny_rows(gpu, rows, cols):
    """Many rows of at most 64 columns take a thread per row (staged through LDS): against float64, the bars
    of the wavefront-per-row kernels; the row count just below the switch gives the same values to rounding."""
    F = gpu.functional
    rng = np.random.default_rng(rows + cols)
    x = (rng.standard_normal((rows, cols)) * 3).astype(np.float32)
    x[5] *= 40                                    # underflowing tail
    if cols > 1:
        x[6, : cols // 2] = -np.inf
    dx = F.from_numpy(x)
    got = F.softmax_fused(dx).numpy()
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(axis=1, keepdims=True))
    want = e / e.sum(axis=1, keepdims=True)
    np.testing.assert_allclose(got, want, rtol=4e-6, atol=1.2e-38)
    few = F.softmax_fused(F.from_numpy(x[:300])).numpy()      # wavefront form
    np.testing.assert_allclose(got[:300], few, rtol=1e-6, atol=1.2e-38)
    # in place
    inplace = F.from_numpy(x)
    F.softmax_fused(inplace, out=inplace)
    np.testing.assert_array_equal(inplace.numpy(), got)
    # rows 1 ... of a tensor with one more row: the run starts off a 16-byte boundary unless cols % 4 == 0
    taller = F.from_numpy(np.concatenate([x[:1], x]))
    np.testing.assert_array_equal(F.softmax_fused(taller.view((1, rows + 1), True)).numpy(), got)
    # LayerNorm
    xl = rng.standard_normal((rows, cols)).astype(np.float32) * 2 + 1
    g = rng.standard_normal(cols).astype(np.float32)
    b = rng.standard_normal(cols).astype(np.float32)
    got = F.layer_norm_fused(F.from_numpy(xl), F.from_numpy(g), F.from_numpy(b), eps=1e-5).numpy()
    x64 = xl.astype(np.float64)
    mean = x64.mean(axis=1, keepdims=True)
    var = ((x64 - mean) ** 2).mean(axis=1, keepdims=True)
    want = (x64 - mean) / np.sqrt(var + np.float64(np.float32(1e-5))) * g + b
    # the deviation x - mean is rounded in binary32: an absolute error of about 2^-24 |x| / std per element
    scale = np.abs(x64).max(axis=1, keepdims=True) / np.sqrt(var + 1e-5)
    assert np.all(np.abs(got - want) <= 4e-7 * scale * np.abs(g) + 2e-6 * np.abs(want) + 1e-6)


@pytest.mark.parametrize("cols", [10, 64])
def test_layernorm_tiny_rows_against_the_wavefront_form_and_its_own_backward(gpu, cols):
    """The thread-per-row LayerNorm starts at 16384 rows.  The same rows through it (16384 rows) and through the
    wavefront form (16383 rows) agree to the rounding of the row statistics, both agree with the reference's
    ten-node recipe (source/nn/norms.lisp:72-82) run node for node, and the backward kernel of the same regime
    recomputes exactly the x-hat the forward produced: with gamma = 1, beta = 0 the forward output is x-hat, and
    with dy a single 1 the gradient of gamma is that row's x-hat."""
    F = gpu.functional
    rng = np.random.default_rng(cols)
    x = (rng.standard_normal((16384, cols)) * 2 + 1).astype(np.float32)
    g = rng.standard_normal(cols).astype(np.float32)
    b = rng.standard_normal(cols).astype(np.float32)
    dg, db = F.from_numpy(g), F.from_numpy(b)
    tiny = F.layer_norm_fused(F.from_numpy(x), dg, db, eps=1e-5).numpy()
    wave = F.layer_norm_fused(F.from_numpy(x[:16383]), dg, db, eps=1e-5).numpy()
    nodes = F.layer_norm(F.from_numpy(x[:2000]), dg, db, eps=1e-5).numpy()
    x64 = x.astype(np.float64)
    std = np.sqrt(x64.var(axis=1, keepdims=True) + 1e-5)
    scale = np.abs(x64).max(axis=1, keepdims=True) / std
    bar = 6e-7 * scale * np.abs(g) + 3e-6 * np.abs(tiny) + 1e-6
    assert np.all(np.abs(tiny[:16383] - wave) <= bar[:16383])
    assert np.all(np.abs(tiny[:2000] - nodes) <= 4 * bar[:2000])
    ones, zeros = F.from_numpy(np.ones(cols, np.float32)), F.from_numpy(np.zeros(cols, np.float32))
    xh = F.layer_norm_fused(F.from_numpy(x), ones, zeros, eps=1e-5).numpy()
    for row in (0, 777, 16383):
        dy = np.zeros_like(x)
        dy[row] = 1.0
        _, dgamma, dbeta = F.layer_norm_backward(F.from_numpy(x), ones, F.from_numpy(dy), 1e-5)
        np.testing.assert_array_equal(dgamma.numpy().ravel(), xh[row])
        np.testing.assert_array_equal(dbeta.numpy().ravel(), np.ones(cols, np.float32))


@pytest.mark.parametrize("seed", range(40))
def test_random_sums_and_selections(gpu, seed):
    """Random shapes (a few long axes, many short ones) and random kept / reduced axes: !sum, !mean, !max and
    argmax against float64 / numpy, on :float and, for the sums, on :double and :int32 too.  Whatever kernel
    the dispatcher picks (rows, tiny rows, columns, narrow columns, middle axes, pieces of long reductions)
    must agree."""
    W = gpu
    F = W.functional
    rng = np.random.default_rng(5000 + seed)
    extents = [1, 2, 3, 4, 7, 10, 32, 33, 64, 100, 128, 129, 1000, 4099, 20000, 70000]
    rank = int(rng.integers(1, 5))
    while True:
        shape = [int(rng.choice(extents)) for _ in range(rank)]
        if 1 <= np.prod(shape) <= 3000000:
            break
    x = (rng.standard_normal(shape) * 2).astype(np.float32)
    dx = F.from_numpy(x)
    x64 = x.astype(np.float64)
    naxes = int(rng.integers(1, rank + 1))
    axes = tuple(sorted(int(a) for a in rng.choice(rank, naxes, replace=False)))
    what = f"{shape} over {axes}"
    got = F.sum(dx, axis=axes if len(axes) > 1 else axes[0]).numpy().reshape(-1)
    want = x64.sum(axis=axes).reshape(-1)
    bar = 2e-6 * np.abs(x64).sum(axis=axes).reshape(-1) + 1e-30
    assert np.all(np.abs(got - want) <= bar), what
    got = F.mean(dx, axis=axes if len(axes) > 1 else axes[0]).numpy().reshape(-1)
    count = np.prod([shape[a] for a in axes])
    assert np.all(np.abs(got - want / count) <= bar / count + 1e-30), what
    # !max / !argmax reduce the trailing `t` axes as one run ((butlast (shape tensor) t) is kept)
    t = int(rng.integers(1, rank + 1))
    runs = x.reshape(shape[:rank - t] + [-1]) if t < rank else x.reshape(1, -1)
    got_max = F.max(dx, axis=t).numpy().reshape(-1) if t < rank else F.max(F.reshape(dx, 1, -1)).numpy().reshape(-1)
    assert_bit_equal(got_max, runs.max(axis=-1).reshape(-1), f"max of the trailing {t} axes, {what}")
    got_arg = (F.argmax(dx, axis=t) if t < rank else F.argmax(F.reshape(dx, 1, -1))).numpy().reshape(-1).astype(np.int64)
    np.testing.assert_array_equal(got_arg, runs.argmax(axis=-1).reshape(-1))   # the first maximum
    xd = F.from_numpy(x64, dtype="double")
    got = F.sum(xd, axis=axes if len(axes) > 1 else axes[0]).numpy().reshape(-1)
    assert np.all(np.abs(got - want) <= 1e-13 * np.abs(x64).sum(axis=axes).reshape(-1) + 1e-300), what
    xi = rng.integers(-2 ** 31, 2 ** 31, shape).astype(np.int32)
    got = F.sum(F.from_numpy(xi, dtype="int32"), axis=axes if len(axes) > 1 else axes[0]).numpy().reshape(-1)
    np.testing.assert_array_equal(got, xi.astype(np.int64).sum(axis=axes).astype(np.int32).reshape(-1))
