"""Row softmax, softmax gradient and argmax on the GPU through the scheduler entries
(mograd/runtime/__init__.mojo:402-405 and the softmax rules) against the oracle.

softmax / softmax_grad are fp32 row reductions: rtol 1e-4 / atol 1e-5 (16-bit storage: the
storage type's rounding).  argmax is index work: bit-exact, including the tie rule (lowest
index), NaN handling and the index being stored in the tensor's float dtype.
"""
import numpy as np
import pytest

from helpers import ATOL_F32, RTOL_F32, assert_close, integers, normal
from oracle import oracle_np as O

pytestmark = pytest.mark.gpu

from mograd_amd import BF16, F16, F32, AnyBuffer, Layout, Node  # noqa: E402
from mograd_amd import runtime as R  # noqa: E402
from mograd_amd.runtime import round_to_dtype  # noqa: E402


def _run(device, op, out_layout, operands, dtype, attrs=None):
    srcs = [Node.leaf(l, dtype) for _, l in operands]
    node = Node(op, out_layout, dtype, srcs, attrs or {})
    bufs = [AnyBuffer.from_numpy(device, a, dtype) for a, _ in operands]
    (out,) = R.run(node, bufs, device)
    return out.to_numpy(out_layout.shape())


SHAPES = [(4, 10), (1, 1), (7, 5), (64, 256), (33, 1000), (3, 5, 64), (2, 12, 96, 96), (16, 4099)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype,rtol,atol", [(F32, RTOL_F32, ATOL_F32), (F16, 2e-3, 1e-4), (BF16, 1.6e-2, 1e-3)])
def test_softmax_and_grad(device, shape, dtype, rtol, atol):
    x = round_to_dtype(normal(90, 0, shape, std=3.0), dtype)
    up = round_to_dtype(normal(90, 1, shape), dtype)
    layout = Layout(*shape)
    y = _run(device, "SOFTMAX", layout, [(x, layout)], dtype)
    assert_close(y, O.softmax(x), rtol, atol, "softmax")
    np.testing.assert_allclose(y.astype(np.float64).sum(-1), 1.0, atol=shape[-1] * (2.0 ** -24 if dtype == F32 else 2.0 ** -9))
    yr = round_to_dtype(O.softmax(x).astype(np.float32), dtype)
    g = _run(device, "SOFTMAX_GRAD", layout, [(yr, layout), (up, layout)], dtype)
    assert_close(g, O.softmax_grad(yr, up), rtol, atol, "softmax_grad")


def test_softmax_extremes(device):
    # rows with huge offsets, a row of -inf except one entry, equal entries
    x = np.array([[1000.0, 1001.0, 999.0, 1000.5], [-1e30, 5.0, -1e30, -1e30], [2.0, 2.0, 2.0, 2.0],
                  [-np.inf, 0.0, -np.inf, 1.0]], dtype=np.float32)
    y = _run(device, "SOFTMAX", Layout(4, 4), [(x, Layout(4, 4))], F32)
    assert np.isfinite(y).all()
    assert_close(y, O.softmax(x), RTOL_F32, ATOL_F32, "softmax extremes")


@pytest.mark.parametrize("dtype", [F32, F16, BF16])
@pytest.mark.parametrize("shape,axis", [((64, 10), 1), ((2048, 10), -1), ((7, 200), 1), ((6, 7, 5), 0), ((6, 7, 5), 1),
                                        ((6, 7, 5), 2), ((1, 1), 1), ((3, 65), 1)])
def test_argmax_exact_with_ties(device, dtype, shape, axis):
    # small integers: many exact ties, all representable in every float dtype
    a = integers(91, 0, shape, -3, 4, np.int32).astype(np.float32)
    out_shape = tuple(s for i, s in enumerate(shape) if i != axis % len(shape))
    got = _run(device, "ARGMAX", Layout(*out_shape), [(a, Layout(*shape))], dtype, {"axis": axis})
    want = O.argmax_axis(a, axis)
    np.testing.assert_array_equal(got, want.astype(np.float32))
    np.testing.assert_array_equal(want, np.argmax(a, axis=axis))


def test_argmax_nan_and_full_reduction(device):
    a = np.array([[np.nan, 1.0, 3.0, 3.0], [np.nan, np.nan, np.nan, np.nan], [-np.inf, -np.inf, -np.inf, -np.inf],
                  [2.0, np.nan, 5.0, np.nan]], dtype=np.float32)
    got = _run(device, "ARGMAX", Layout(4), [(a, Layout(4, 4))], F32, {"axis": 1})
    np.testing.assert_array_equal(got, [2.0, 0.0, 0.0, 2.0])
    # no axis: the whole tensor is one lane (kernels/reduce.mojo:181-203)
    b = normal(92, 0, (37, 11))
    got = _run(device, "ARGMAX", Layout(1), [(b, Layout(37, 11))], F32)
    assert int(got[0]) == int(np.argmax(b))


def test_accuracy_of_a_batch(device):
    # the training loops' metric: argmax over 10 logits per row for 2048 rows, compared with labels
    logits = normal(93, 0, (2048, 10))
    pred = _run(device, "ARGMAX", Layout(2048), [(logits, Layout(2048, 10))], F32, {"axis": 1})
    np.testing.assert_array_equal(pred.astype(np.int64), np.argmax(logits, axis=1))
