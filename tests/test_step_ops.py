"""The remaining per-step ops of a transformer block on the GPU: add, relu, cast,
contiguous, gather and scatter_add, through the scheduler entries the reference's graph
reaches (mograd/runtime/__init__.mojo:239-256,296-333,456-461).

add / relu / contiguous / gather move or combine values with at most one rounding, so
they are checked bit for bit against numpy on the same (already rounded) inputs.
scatter_add is a sum: it is checked against the float64 oracle at the fp32-reduction
tolerance, for run-to-run bit equality (it uses no atomics), and through the adjoint
identity with gather at full size.
"""
import numpy as np
import pytest

from helpers import ATOL_F32, RTOL_F32, assert_close, assert_sum_close, integers, normal
from oracle import oracle_np as O

pytestmark = pytest.mark.gpu

from mograd_amd import BF16, F16, F32, I32, I64, AnyBuffer, Layout, MogradError, Node  # noqa: E402
from mograd_amd import runtime as R  # noqa: E402
from mograd_amd.runtime import round_to_dtype  # noqa: E402

FLOATS = [F32, F16, BF16]


def _run(device, op, out_layout, operands, dtype=F32, attrs=None):
    """operands: list of (host array, layout view, dtype)."""
    srcs = [Node.leaf(l, d) for _, l, d in operands]
    node = Node(op, out_layout, dtype, srcs, attrs or {})
    bufs = [AnyBuffer.from_numpy(device, a, d).view(l) for a, l, d in operands]
    (out,) = R.run(node, bufs, device)
    return out.to_numpy(out_layout.shape())


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("n", [1, 7, 8, 1000, 4096, 1 << 20, (1 << 20) + 3])
def test_add_relu_exact(device, dtype, n):
    a = round_to_dtype(normal(60, 0, (n,)), dtype)
    b = round_to_dtype(normal(60, 1, (n,)), dtype)
    got = _run(device, "ADD", Layout(n), [(a, Layout(n), dtype), (b, Layout(n), dtype)], dtype)
    # one fp32 add, one rounding to the storage type
    np.testing.assert_array_equal(got, round_to_dtype(a + b, dtype))
    got = _run(device, "RELU", Layout(n), [(a, Layout(n), dtype)], dtype)
    np.testing.assert_array_equal(got, np.maximum(a, 0))


@pytest.mark.parametrize("src,dst", [(F32, BF16), (F32, F16), (BF16, F32), (F16, F32), (F16, BF16), (BF16, F16),
                                     (F32, F32)])
@pytest.mark.parametrize("n", [5, 8, 4099, 1 << 18])
def test_cast_single_rounding(device, src, dst, n):
    a = round_to_dtype(normal(61, 0, (n,), std=3.0), src)
    a[:3] = [0.0, 1.0 + 2.0 ** -8, -60000.0][: min(3, n)]  # 1 + 2^-8 is a rounding tie for bf16
    a = round_to_dtype(a, src)
    got = _run(device, "CAST", Layout(n), [(a, Layout(n), src)], dst)
    np.testing.assert_array_equal(got, round_to_dtype(a, dst))


CONTIG_CASES = [
    # shape of the view, strides of the view (elements), size of the backing array
    ((4, 6), (1, 4), 24),                        # transpose of (6, 4)
    ((2, 5, 3, 8), (120, 8, 40, 1), 240),        # BHSD buffer read as BSHD: (B,S,H,D) view
    ((2, 3, 5, 8), (120, 8, 24, 1), 240),        # BSHD buffer read as BHSD
    ((3, 4, 16), (0, 16, 1), 64),                # broadcast leading dim
    ((5, 7), (14, 2), 70),                       # every other column
    ((2, 3, 4), (12, 4, 1), 24),                 # already contiguous
    ((6,), (3,), 18),
    ((1, 1), (1, 1), 1),
    # transposes long enough for the tiled kernel (one dim contiguous in the source, the innermost strided)
    ((100, 70), (1, 100), 7000),                 # plain 2-D transpose, ragged tiles
    ((64, 128), (1, 64), 8192),                  # whole tiles
    ((3, 50, 40), (2000, 1, 50), 6000),          # batched transpose
    ((33, 5, 47), (1, 33, 165), 33 * 5 * 47),    # dims reversed: a batch dim between the two
    ((2, 40, 3, 36), (40, 1, 2880, 80), 8640),   # batch dims outside and between, a permuted 4-D tensor
    ((48, 20), (2, 100), 2000),                  # strided both ways: not a transpose, element by element
    ((40, 33), (1, 80), 80 * 33),                # a transposed slice: rows of the source 80 apart
]


@pytest.mark.parametrize("shape,strides,backing", CONTIG_CASES)
@pytest.mark.parametrize("dtype", [F32, BF16, I64, I32])
def test_contiguous_matches_numpy_view(device, shape, strides, backing, dtype):
    if dtype in (I64, I32):
        base = integers(62, 0, (backing,), -1000, 1000, np.int64 if dtype == I64 else np.int32)
    else:
        base = round_to_dtype(normal(62, 0, (backing,)), dtype)
    item = base.itemsize
    want = np.lib.stride_tricks.as_strided(base, shape, tuple(s * item for s in strides))
    view = Layout(*shape, strides=strides)
    got = _run(device, "CONTIGUOUS", Layout(*shape), [(base, view, dtype)], dtype)
    np.testing.assert_array_equal(got, want)


def test_contiguous_attention_layout_full_size(device):
    # O (B, H, S, D) -> (B, S, H, D) at the GPT step's size, bf16
    B, H, S, D = 64, 6, 256, 64
    o = round_to_dtype(normal(63, 0, (B, H, S, D)), BF16)
    view = Layout(B, H, S, D).transpose(1, 2)
    got = _run(device, "CONTIGUOUS", Layout(B, S, H, D), [(o, view, BF16)], BF16)
    np.testing.assert_array_equal(got, o.transpose(0, 2, 1, 3))


def test_contiguous_rejects_bad_rank(device):
    buf = AnyBuffer.create(F32, device, 4)
    with pytest.raises(MogradError):
        device.lib.mg_contiguous(buf.data_ptr(), buf.data_ptr(), 9, R._i64_array([1] * 9), R._i64_array([1] * 9), F32,
                                 device.stream)


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("idx_dtype", [I32, I64])
@pytest.mark.parametrize("V,d,idx_shape", [(65, 384, (4, 33)), (7, 5, (11,)), (1000, 64, (2, 3, 5)), (3, 8, (1,))])
def test_gather_rows_exact(device, dtype, idx_dtype, V, d, idx_shape):
    w = round_to_dtype(normal(64, 0, (V, d)), dtype)
    idx = integers(64, 1, idx_shape, 0, V, np.int32 if idx_dtype == I32 else np.int64)
    got = _run(device, "GATHER", Layout(*idx_shape, d), [(w, Layout(V, d), dtype), (idx, Layout(*idx_shape), idx_dtype)],
               dtype)
    np.testing.assert_array_equal(got, w[idx])


def test_gather_strided_source_and_bad_index(device):
    V, d = 9, 12
    wt = normal(65, 0, (d, V))  # the source is the transposed view of this array
    idx = np.array([0, 8, 3, 3, -1, 9], dtype=np.int64)
    got = _run(device, "GATHER", Layout(6, d), [(wt, Layout(d, V).transpose(), F32), (idx, Layout(6), I64)], F32)
    np.testing.assert_array_equal(got[:4], wt.T[idx[:4]])
    assert not got[4:].any()  # out-of-range rows come back as zeros
    with pytest.raises(MogradError):  # op.mojo:367-368
        _run(device, "GATHER", Layout(6, d), [(wt, Layout(d * V), F32), (idx, Layout(6), I64)], F32)


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("idx_dtype", [I32, I64])
@pytest.mark.parametrize("V,d,n", [(65, 384, 4096), (7, 5, 40), (1000, 64, 300), (3, 8, 1), (50, 136, 5000)])
def test_scatter_add_vs_oracle(device, dtype, idx_dtype, V, d, n):
    y = round_to_dtype(normal(66, 0, (n, d)), dtype)
    idx = integers(66, 1, (n,), 0, V, np.int32 if idx_dtype == I32 else np.int64)
    operands = [(idx, Layout(n), idx_dtype), (y, Layout(n, d), dtype)]
    got = _run(device, "SCATTER_ADD", Layout(V, d), operands, dtype)
    want = O.scatter_add(idx, y, V)
    mass = O.scatter_add(idx, np.abs(y), V)
    if dtype == F32:
        assert_sum_close(got, want, mass, what="scatter_add")
    else:
        # fp32 accumulation, then one rounding to the 16-bit output
        eps = 2.0 ** -8 if dtype == BF16 else 2.0 ** -11
        assert np.all(np.abs(got - want) <= eps * np.abs(want) + 16 * 2.0 ** -24 * mass + 1e-30)
    again = _run(device, "SCATTER_ADD", Layout(V, d), operands, dtype)
    np.testing.assert_array_equal(got, again)  # no atomics: bit-identical on every run
    untouched = np.setdiff1d(np.arange(V), idx)
    assert not got[untouched].any()


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("idx_dtype", [I32, I64])
@pytest.mark.parametrize("V,d,n", [(2048, 64, 3000), (5000, 72, 700), (1024, 5, 1)])
def test_scatter_add_large_table_buckets(device, monkeypatch, dtype, idx_dtype, V, d, n):
    # From a thousand rows on the indices are bucketed by destination row (a stable sort of
    # (row, position) pairs) and a wave adds only its own row's run, in the same ascending
    # position order as the scanning kernel: forcing either path gives the same bits.  Indices
    # outside the table, repeated heavily and absent rows are all in the mix.
    y = round_to_dtype(normal(70, 0, (n, d)), dtype)
    idx = integers(70, 1, (n,), -3, V + 3, np.int32 if idx_dtype == I32 else np.int64)
    idx[: n // 4] = idx[0] if 0 <= idx[0] < V else 7  # one heavy row
    operands = [(idx, Layout(n), idx_dtype), (y, Layout(n, d), dtype)]
    monkeypatch.setenv("MOGRAD_HIP_SCATTER_BUCKET_MIN_ROWS", "1")
    got = _run(device, "SCATTER_ADD", Layout(V, d), operands, dtype)
    keep = (idx >= 0) & (idx < V)
    want = O.scatter_add(idx[keep], y[keep], V)
    mass = O.scatter_add(idx[keep], np.abs(y[keep]), V)
    eps = {F32: 0.0, F16: 2.0 ** -11, BF16: 2.0 ** -8}[dtype]
    assert np.all(np.abs(got - want) <= RTOL_F32 * np.abs(want) + eps * np.abs(want) + 16 * 2.0 ** -24 * mass + 1e-30)
    assert not got[np.setdiff1d(np.arange(V), idx[keep])].any()
    if n <= 1024:  # one slab of the scanning kernel: the same order of additions
        monkeypatch.setenv("MOGRAD_HIP_SCATTER_BUCKET_MIN_ROWS", "1000000000")
        np.testing.assert_array_equal(got, _run(device, "SCATTER_ADD", Layout(V, d), operands, dtype))


def test_scatter_add_vocabulary_sized_table(device):
    # A GPT-2 embedding gradient: 8192 tokens into (50304, 768) bf16.  Histogram exactly, the
    # adjoint identity with gather, untouched rows zero, two runs identical.
    V, d, n = 50304, 768, 8192
    idx = integers(71, 0, (n,), 0, V, np.int32)
    idx[:512] = 11  # a frequent token
    y = round_to_dtype(normal(71, 1, (n, d)), BF16)
    operands = [(idx, Layout(n), I32), (y, Layout(n, d), BF16)]
    got = _run(device, "SCATTER_ADD", Layout(V, d), operands, BF16)
    np.testing.assert_array_equal(got, _run(device, "SCATTER_ADD", Layout(V, d), operands, BF16))
    assert not got[np.setdiff1d(np.arange(V), idx)].any()
    rows = np.unique(idx)[:200]
    want = O.scatter_add(idx, y, V)[rows]
    assert np.all(np.abs(got[rows] - want) <= 2.0 ** -8 * np.abs(want) + 1e-3)
    ones = np.ones((n, 8), np.float32)
    hist = _run(device, "SCATTER_ADD", Layout(V, 8), [(idx, Layout(n), I32), (ones, Layout(n, 8), F32)], F32)
    np.testing.assert_array_equal(hist[:, 0], np.bincount(idx, minlength=V).astype(np.float32))


@pytest.mark.parametrize("max_tiles", [16384, 5, 1])
@pytest.mark.parametrize("idx_dtype", [I32, I64])
@pytest.mark.parametrize("V,n", [(70000, 200000), (300, 1031), (65536, 40000), (1 << 16 | 1, 9000)])
def test_scatter_add_sort_places_every_pair_once(device, monkeypatch, idx_dtype, V, n, max_tiles):
    # The bucketing sort is a radix sort of (row, position) pairs, eight bits a pass: tables of
    # up to 256, 65536 and more rows take one, two and three passes, a list of more than 1024
    # pairs takes several tiles, and the tile limit lowered to 5 and 1 makes a thread carry more
    # than four pairs.  Small integer values sum exactly in fp32 in any order, so the result
    # equals the oracle's bit for bit only if every pair reached its own row exactly once.
    d = 8
    y = integers(72, 0, (n, d), -8, 9, np.int32).astype(np.float32)
    idx = integers(72, 1, (n,), -2, V + 2, np.int32 if idx_dtype == I32 else np.int64)
    idx[: n // 8] = V - 1  # one heavy row, in the last bucket of every pass
    keep = (idx >= 0) & (idx < V)
    monkeypatch.setenv("MOGRAD_HIP_SCATTER_BUCKET_MIN_ROWS", "1")
    monkeypatch.setenv("MOGRAD_HIP_SCATTER_RANGE_READS_LOG2", "0")  # the sort, whatever the list's length
    monkeypatch.setenv("MOGRAD_HIP_SCATTER_SORT_MAX_TILES", str(max_tiles))
    got = _run(device, "SCATTER_ADD", Layout(V, d), [(idx, Layout(n), idx_dtype), (y, Layout(n, d), F32)], F32)
    np.testing.assert_array_equal(got, O.scatter_add(idx[keep], y[keep], V).astype(np.float32))


@pytest.mark.parametrize("areas", [-1, 1, 0])
@pytest.mark.parametrize("idx_dtype", [I32, I64])
@pytest.mark.parametrize("V,d,n,heavy", [(50304, 8, 8192, 512), (70000, 8, 5000, 3000), (300, 24, 1031, 128),
                                         (4096 * 9 + 5, 8, 1, 0), (2048, 520, 2500, 2500), (65, 8, 700, 0)])
def test_scatter_add_row_ranges_place_every_pair_once(device, monkeypatch, idx_dtype, V, d, n, heavy, areas):
    # Short lists into large tables take one launch: a workgroup per range of rows collects the
    # pairs of its rows from the whole list.  A row that more than 512 pairs of one quarter of
    # the list point at makes its workgroup keep its lists in global memory instead of LDS; the
    # last range of a table is shorter than the others; 520 columns leave the second column
    # block mostly empty.  With one area for the two workgroups that need one, or none, the
    # workgroups left without read the whole list once per row.  Exact for the same reason as above.
    y = integers(73, 0, (n, d), -8, 9, np.int32).astype(np.float32)
    idx = integers(73, 1, (n,), -2, V + 2, np.int32 if idx_dtype == I32 else np.int64)
    idx[:heavy] = V - 1
    keep = (idx >= 0) & (idx < V)
    monkeypatch.setenv("MOGRAD_HIP_SCATTER_BUCKET_MIN_ROWS", "1")
    monkeypatch.setenv("MOGRAD_HIP_SCATTER_RANGE_READS_LOG2", "30")
    if areas >= 0:
        monkeypatch.setenv("MOGRAD_HIP_SCATTER_SPILL_SLOTS", str(areas))
    got = _run(device, "SCATTER_ADD", Layout(V, d), [(idx, Layout(n), idx_dtype), (y, Layout(n, d), F32)], F32)
    np.testing.assert_array_equal(got, O.scatter_add(idx[keep], y[keep], V).astype(np.float32))


@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("V,d,n", [(2048, 64, 3000), (50304, 136, 4000)])
def test_scatter_add_forms_agree_bit_for_bit(device, monkeypatch, dtype, V, d, n):
    # Row ranges, the sort and (one slab) the scanning kernel all add a row's values in
    # ascending position order in fp32 from zero: the same bits, with and without streaming stores.
    y = round_to_dtype(normal(74, 0, (n, d)), dtype)
    idx = integers(74, 1, (n,), -3, V + 3, np.int32)
    idx[: n // 3] = 17
    operands = [(idx, Layout(n), I32), (y, Layout(n, d), dtype)]
    monkeypatch.setenv("MOGRAD_HIP_SCATTER_RANGE_READS_LOG2", "30")
    ranges = _run(device, "SCATTER_ADD", Layout(V, d), operands, dtype)
    monkeypatch.setenv("MOGRAD_HIP_SCATTER_STREAM", "0")
    np.testing.assert_array_equal(ranges, _run(device, "SCATTER_ADD", Layout(V, d), operands, dtype))
    monkeypatch.setenv("MOGRAD_HIP_SCATTER_RANGE_READS_LOG2", "0")
    np.testing.assert_array_equal(ranges, _run(device, "SCATTER_ADD", Layout(V, d), operands, dtype))
    if n <= 1024 * 3 and V <= 2048:
        monkeypatch.setenv("MOGRAD_HIP_SCATTER_BUCKET_MIN_ROWS", "1000000000")
        # several slabs here: partial sums are regrouped, so only to the summation tolerance
        scan = _run(device, "SCATTER_ADD", Layout(V, d), operands, dtype)
        eps = {F32: 2.0 ** -20, F16: 2.0 ** -10, BF16: 2.0 ** -7}[dtype]
        assert np.all(np.abs(scan - ranges) <= eps * (np.abs(ranges) + 64.0))


def test_scatter_add_ignores_bad_indices_and_checks_rank(device):
    V, d, n = 5, 8, 6
    y = normal(67, 0, (n, d))
    idx = np.array([0, 4, -1, 5, 4, 100], dtype=np.int64)
    got = _run(device, "SCATTER_ADD", Layout(V, d), [(idx, Layout(n), I64), (y, Layout(n, d), F32)], F32)
    keep = (idx >= 0) & (idx < V)
    assert_close(got, O.scatter_add(idx[keep], y[keep], V), RTOL_F32, ATOL_F32, "scatter_add")
    with pytest.raises(MogradError):  # op.mojo:375-376
        _run(device, "SCATTER_ADD", Layout(V, d), [(idx, Layout(n), I64), (y, Layout(n * d), F32)], F32)


def test_embedding_grad_adjoint_full_size(device):
    # GPT step size: 16384 tokens, vocab 65, d 384.  <gather(W, i), Y> = <W, scatter_add(i, Y)>
    # ties the two kernels to each other without a CPU loop over tokens.
    V, d, n = 65, 384, 16384
    w = normal(68, 0, (V, d))
    y = normal(68, 1, (n, d))
    idx = integers(68, 2, (n,), 0, V, np.int32)
    g = _run(device, "GATHER", Layout(n, d), [(w, Layout(V, d), F32), (idx, Layout(n), I32)], F32)
    sa = _run(device, "SCATTER_ADD", Layout(V, d), [(idx, Layout(n), I32), (y, Layout(n, d), F32)], F32)
    lhs = np.sum(g.astype(np.float64) * y)
    rhs = np.sum(w.astype(np.float64) * sa)
    mass = np.sum(np.abs(g.astype(np.float64) * y))
    assert abs(lhs - rhs) <= RTOL_F32 * abs(lhs) + 16 * 2.0 ** -24 * mass
    # and the counts: scattering ones gives the histogram of the indices, exactly
    ones = np.ones((n, 8), np.float32)
    hist = _run(device, "SCATTER_ADD", Layout(V, 8), [(idx, Layout(n), I32), (ones, Layout(n, 8), F32)], F32)
    np.testing.assert_array_equal(hist[:, 0], np.bincount(idx, minlength=V).astype(np.float32))


MAP_VIEWS = [
    # shape, strides of operand a, strides of operand b, elements behind a, behind b
    ((64, 48), (1, 64), (48, 1), 64 * 48, 64 * 48),                 # a transposed, b row-major
    ((40, 96), (96, 1), (0, 1), 40 * 96, 96),                        # b a bias row broadcast over the rows
    ((40, 96), (96, 1), (1, 0), 40 * 96, 40),                        # b a column broadcast along the rows
    ((2, 5, 3, 16), (240, 16, 80, 1), (240, 48, 16, 1), 480, 480),   # a (B,H,S,D) read as (B,S,H,D)
    ((6, 24), (48, 2), (24, 1), 6 * 48, 6 * 24),                     # every other column of a
    ((3, 4, 32), (0, 32, 1), (128, 32, 1), 128, 384),                # a broadcast over the leading dim
    ((7, 9), (9, 1), (0, 0), 63, 1),                                 # b one value
    ((5, 8), (12, 1), (8, 1), 60, 40),                               # rows of a 12 apart: 16-byte rows in fp32, not in 16 bits
    ((1 << 12, 1 << 7), (1 << 7, 1), (0, 1), 1 << 19, 1 << 7),       # large, bias
    ((1 << 10, 1 << 9), (1, 1 << 10), (1 << 9, 1), 1 << 19, 1 << 19),  # large, transposed
    ((13,), (3,), (1,), 39, 13),
    ((1, 1), (1, 1), (1, 1), 1, 1),
]


@pytest.mark.parametrize("shape,sa,sb,na,nb", MAP_VIEWS)
@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("offset", [0, 1])
def test_maps_over_strided_views(device, shape, sa, sb, na, nb, dtype, offset):
    # add, relu, relu_grad and cast read strided views themselves (the reference's *_strided
    # kernels, kernels/strided.mojo:54-114): transposed, sliced and broadcast operands, at 16-byte
    # aligned and at odd base offsets.  One rounding at most, so the results are compared bit for
    # bit with numpy on the same views.
    a = round_to_dtype(normal(75, 0, (na + offset,)), dtype)
    b = round_to_dtype(normal(75, 1, (nb + offset,)), dtype)
    item = a.itemsize
    va = np.lib.stride_tricks.as_strided(a[offset:], shape, tuple(t * item for t in sa))
    vb = np.lib.stride_tricks.as_strided(b[offset:], shape, tuple(t * item for t in sb))
    la = Layout(*shape, strides=sa, base_offset=offset)
    lb = Layout(*shape, strides=sb, base_offset=offset)
    out = Layout(*shape)
    got = _run(device, "ADD", out, [(a, la, dtype), (b, lb, dtype)], dtype)
    np.testing.assert_array_equal(got, round_to_dtype(va + vb, dtype))
    got = _run(device, "RELU_GRAD", out, [(a, la, dtype), (b, lb, dtype)], dtype)
    np.testing.assert_array_equal(got, np.where(va > 0, vb, 0).astype(np.float32))
    got = _run(device, "RELU", out, [(a, la, dtype)], dtype)
    np.testing.assert_array_equal(got, np.maximum(va, 0))
    for to in FLOATS:
        got = _run(device, "CAST", out, [(a, la, dtype)], to)
        np.testing.assert_array_equal(got, round_to_dtype(va, to))


SOFTMAX_VIEWS = [
    # shape, strides, elements behind the view
    ((48, 64), (1, 48), 48 * 64),                    # transposed: a row runs down a column
    ((2, 5, 3, 16), (240, 16, 80, 1), 480),          # permuted heads, contiguous rows of 16
    ((6, 24), (48, 2), 6 * 48),                      # every other column
    ((3, 4, 32), (0, 32, 1), 128),                   # broadcast leading dim
    ((5, 40), (56, 1), 5 * 56),                      # rows with a gap between them
    ((7,), (3,), 21),
    ((300, 1000), (1000, 1), 300000),                # contiguous, through the strided entry at an odd offset
    ((512, 256), (1, 512), 512 * 256),               # a large transpose: copied through the tiled transpose first
]


@pytest.mark.parametrize("shape,strides,n", SOFTMAX_VIEWS)
@pytest.mark.parametrize("dtype", FLOATS)
@pytest.mark.parametrize("offset", [0, 3])
def test_softmax_over_strided_views(device, shape, strides, n, dtype, offset):
    # SOFTMAX of a view runs mograd_softmax_strided in the reference (kernels/__init__.mojo:1033-1060)
    # and mg_softmax_strided here: the same arithmetic as the contiguous kernel, so it must agree
    # with the contiguous kernel on a row-major copy of the view, and with the oracle, within the
    # storage type's rounding.
    a = round_to_dtype(normal(76, 0, (n + offset,), std=2.0), dtype)
    view = np.lib.stride_tricks.as_strided(a[offset:], shape, tuple(t * a.itemsize for t in strides))
    layout = Layout(*shape, strides=strides, base_offset=offset)
    lib, st = device.lib, device.stream
    buf = AnyBuffer.from_numpy(device, a, dtype).view(layout)
    got = AnyBuffer.create(dtype, device, view.size)
    lib.mg_softmax_strided(buf.data_ptr(), got.data_ptr(), len(shape), R._i64_array(shape), R._i64_array(strides), dtype, st)
    flat = AnyBuffer.from_numpy(device, np.ascontiguousarray(view), dtype)
    ref = AnyBuffer.create(dtype, device, view.size)
    cols = shape[-1]
    lib.mg_softmax(flat.data_ptr(), ref.data_ptr(), view.size // cols, cols, dtype, st)
    # (a view whose rows cannot be read 16 bytes at a time is summed in another order: a few ulps)
    tol = {F32: 1e-6, F16: 1e-3, BF16: 8e-3}[dtype]
    np.testing.assert_allclose(got.to_numpy(shape), ref.to_numpy(shape), rtol=tol, atol=0)
    np.testing.assert_allclose(got.to_numpy(shape), O.softmax(view.astype(np.float64)), rtol=tol, atol=tol)
    # and through the scheduler entry
    out = _run(device, "SOFTMAX", Layout(*shape), [(a, layout, dtype)], dtype)
    np.testing.assert_array_equal(out, got.to_numpy(shape))


def test_strided_maps_check_their_arguments(device):
    lib, st = device.lib, device.stream
    buf = AnyBuffer.create(F32, device, 64, fill=1.0)
    arr = lambda *v: R._i64_array(v)  # noqa: E731
    with pytest.raises(MogradError, match="rank"):
        lib.mg_relu_strided(buf.data_ptr(), buf.data_ptr(), 9, arr(*[1] * 9), arr(*[1] * 9), F32, st)
    with pytest.raises(MogradError, match="negative"):
        lib.mg_add_strided(buf.data_ptr(), buf.data_ptr(), buf.data_ptr(), 1, arr(8), arr(1), arr(-1), F32, st)
    with pytest.raises(MogradError, match="dtype"):
        lib.mg_cast_strided(buf.data_ptr(), buf.data_ptr(), 1, arr(8), arr(1), F32, I32, st)
    with pytest.raises(MogradError, match="null"):
        lib.mg_relu_grad_strided(buf.data_ptr(), None, buf.data_ptr(), 1, arr(8), arr(1), arr(1), F32, st)
    with pytest.raises(MogradError, match="rank"):
        lib.mg_softmax_strided(buf.data_ptr(), buf.data_ptr(), 0, arr(1), arr(1), F32, st)
    # an empty view is no work, whatever the pointers
    lib.mg_softmax_strided(None, None, 2, arr(0, 8), arr(8, 1), F32, st)
    lib.mg_add_strided(None, None, None, 2, arr(0, 8), arr(8, 1), arr(8, 1), F32, st)


def test_strided_operands_are_materialised(device):
    # Row kernels (axis sums, softmax, argmax) and the index operand of gather take a strided
    # operand through a row-major copy; the elementwise maps read it in place.  Same values either way.
    a = normal(69, 0, (6, 8))
    b = normal(69, 1, (8, 6))
    at = Layout(6, 8).transpose()            # (8, 6) view of a
    got = _run(device, "ADD", Layout(8, 6), [(a, at, F32), (b, Layout(8, 6), F32)], F32)
    np.testing.assert_array_equal(got, a.T + b)
    every_other = Layout(6, 8).slice_axis(1, 0, 8, 2)   # (6, 4), stride (8, 2)
    got = _run(device, "RELU", Layout(6, 4), [(a, every_other, F32)], F32)
    np.testing.assert_array_equal(got, np.maximum(a[:, ::2], 0))
    got = _run(device, "CAST", Layout(8, 6), [(a, at, F32)], BF16)
    np.testing.assert_array_equal(got, round_to_dtype(a.T, BF16))
    up = normal(69, 2, (8, 6))
    got = _run(device, "RELU_GRAD", Layout(8, 6), [(a, at, F32), (up, Layout(8, 6), F32)], F32)
    np.testing.assert_array_equal(got, np.where(a.T > 0, up, 0).astype(np.float32))
    got = _run(device, "SUM", Layout(6), [(a, at, F32)], F32, {"axis": 0})
    np.testing.assert_allclose(got, a.T.sum(axis=0), rtol=1e-5, atol=1e-6)
    got = _run(device, "SOFTMAX", Layout(8, 6), [(a, at, F32)], F32)
    np.testing.assert_allclose(got, O.softmax(a.T), rtol=1e-4, atol=1e-6)
    got = _run(device, "ARGMAX", Layout(8), [(a, at, F32)], F32, {"axis": 1})
    np.testing.assert_array_equal(got, np.argmax(a.T, axis=1).astype(np.float32))
    w = normal(69, 3, (10, 4))
    idx = integers(69, 4, (3, 5), 0, 10, np.int64)
    idx_t = Layout(3, 5).transpose()         # (5, 3) view of the index array
    got = _run(device, "GATHER", Layout(5, 3, 4), [(w, Layout(10, 4), F32), (idx, idx_t, I64)], F32)
    np.testing.assert_array_equal(got, w[idx.T])
