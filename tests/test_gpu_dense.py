"""GPU parity of the dense products and of the activation / loss kernels through the C ABI."""
import pytest
import torch
import torch.nn.functional as F

from tests.util import REL_TOL, gemm_error

pytestmark = pytest.mark.gpu


def _rand(shape, seed):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


SHAPES = [(1, 1, 1), (5, 3, 2), (1000, 602, 16), (777, 16, 41), (300, 128, 16), (4099, 300, 24), (513, 16, 602),
          (130, 41, 16), (2000, 64, 100), (50, 700, 70),
          # span tails of X W (whole steps only, whole + ragged, a single ragged step), row counts off the 16-row tiles,
          # every column-tile count of X^T G, column chunks and all three store widths of G W^T
          (33, 48, 16), (17, 52, 33), (64, 20, 5), (9, 4, 64), (1500, 320, 48), (700, 1024, 64), (600, 603, 20),
          (250, 1000, 64), (4100, 65, 8), (1000, 256, 1)]


@pytest.mark.parametrize("n,k,fo", SHAPES)
def test_dense_xw(cuda, n, k, fo):
    from cagnet_amd import ops
    X, W = _rand((n, k), 1), _rand((k, fo), 2)
    Z = ops.dense_xw(X.to(cuda), W.to(cuda))
    assert gemm_error(Z, X, W) <= REL_TOL
    Zr = ops.dense_xw(X.to(cuda), W.to(cuda), relu=True)
    assert torch.equal(Zr, torch.relu(Z))   # same accumulation, only the store differs


@pytest.mark.parametrize("n,k,fo", SHAPES)
def test_dense_gwt(cuda, n, k, fo):
    from cagnet_amd import ops
    G, W = _rand((n, fo), 3), _rand((k, fo), 4)
    dX = ops.dense_gwt(G.to(cuda), W.to(cuda))
    assert gemm_error(dX, G, W.t()) <= REL_TOL


@pytest.mark.parametrize("n,k,fo", SHAPES + [(100000, 602, 16), (200000, 16, 41)])
def test_dense_xtg(cuda, n, k, fo):
    from cagnet_amd import ops
    X, G = _rand((n, k), 5), _rand((n, fo), 6)
    dW = ops.dense_xtg(X.to(cuda), G.to(cuda))
    assert gemm_error(dW, X.t(), G) <= REL_TOL
    assert torch.equal(dW, ops.dense_xtg(X.to(cuda), G.to(cuda)))  # fixed slice order: bit identical


def test_dense_strided_operands(cuda):
    """Row stride larger than the width (a column slice of a wider matrix) is passed as ld."""
    from cagnet_amd import ops
    big = _rand((300, 700), 7).to(cuda)
    X = big[:, 10:612]                      # 602 wide, ld 700, base not 16-byte aligned
    W = _rand((602, 16), 8).to(cuda)
    assert gemm_error(ops.dense_xw(X, W), X.cpu(), W.cpu()) <= REL_TOL


@pytest.mark.parametrize("n,c", [(1, 1), (7, 8), (1000, 41), (333, 24), (50, 256), (4097, 16), (257, 4), (129, 64),
                                 (1001, 40), (70001, 24)])
def test_log_softmax_and_relu(cuda, n, c):
    from cagnet_amd import ops
    z = (_rand((n, c), 9) * 5.0)
    out = ops.log_softmax_fwd(z.to(cuda))
    ref = F.log_softmax(z.double(), dim=1)
    assert float((out.cpu().double() - ref).abs().max()) <= 1e-5 * max(1.0, float(ref.abs().max()))
    g = _rand((n, c), 10)
    dz = ops.log_softmax_bwd(g.to(cuda), out)
    zr = z.double().requires_grad_(True)
    (F.log_softmax(zr, dim=1) * g.double()).sum().backward()
    scale = g.double().abs().sum(dim=1, keepdim=True)
    assert float(((dz.cpu().double() - zr.grad).abs() / scale.clamp_min(1e-30)).max()) <= REL_TOL
    h = ops.relu_fwd(z.to(cuda))
    assert torch.equal(h.cpu(), torch.relu(z))
    assert torch.equal(ops.relu_bwd(g.to(cuda), h).cpu(), g * (z > 0))


@pytest.mark.parametrize("n,c,frac", [(1, 3, 1.0), (1000, 41, 0.66), (5000, 8, 1.0), (70000, 24, 0.3), (300, 5, 0.0),
                                      (513, 4, 0.5), (999, 64, 1.0), (2000, 40, 0.7), (300, 16, 0.0)])
def test_nll_loss_forward_backward(cuda, n, c, frac):
    from cagnet_amd import ops
    gen = torch.Generator().manual_seed(11)
    logp = F.log_softmax(torch.randn(n, c, generator=gen), dim=1)
    y = torch.randint(0, c, (n,), generator=gen)
    mask = None if frac >= 1.0 else (torch.rand(n, generator=gen) < frac)
    loss, count = ops.nll_loss_fwd(logp.to(cuda), y.to(cuda), None if mask is None else mask.to(cuda))
    sel = slice(None) if mask is None else mask
    expect_count = n if mask is None else int(mask.sum())
    assert int(count) == expect_count
    if expect_count == 0:
        assert float(loss) == 0.0           # the reference's fake_loss branch (gcn_distr.py:359-362)
    else:
        ref = F.nll_loss(logp.double()[sel], y[sel])
        assert abs(float(loss) - float(ref)) <= 1e-5 * max(1.0, abs(float(ref)))
        assert float(loss) == float(ops.nll_loss_fwd(logp.to(cuda), y.to(cuda),
                                                     None if mask is None else mask.to(cuda))[0])
    # gradients: separate kernels and the fused one against autograd
    gs = torch.tensor(0.5)
    d = ops.nll_loss_bwd(y.to(cuda), None if mask is None else mask.to(cuda), count, gs.to(cuda), n, c)
    lp = logp.double().requires_grad_(True)
    if expect_count:
        (F.nll_loss(lp[sel], y[sel]) * 0.5).backward()
        assert float((d.cpu().double() - lp.grad).abs().max()) <= 1e-6
    else:
        assert torch.count_nonzero(d) == 0
    z = torch.randn(n, c, generator=gen)
    out = ops.log_softmax_fwd(z.to(cuda))
    fused = ops.log_softmax_nll_bwd(out, y.to(cuda), None if mask is None else mask.to(cuda), count, gs.to(cuda))
    two_step = ops.log_softmax_bwd(d, out)
    assert float((fused - two_step).abs().max()) <= 1e-6
    if expect_count:
        zr = z.double().requires_grad_(True)
        (F.nll_loss(F.log_softmax(zr, dim=1)[sel], y[sel]) * 0.5).backward()
        assert float((fused.cpu().double() - zr.grad).abs().max()) <= 1e-6
    # forward fused as well: the same log-probabilities, count and (bit for bit) loss as the two calls
    m = None if mask is None else mask.to(cuda)
    logp2, loss2, count2 = ops.log_softmax_nll_fwd(z.to(cuda), y.to(cuda), m)
    loss1, count1 = ops.nll_loss_fwd(out, y.to(cuda), m)
    assert torch.equal(logp2, out) and int(count2) == int(count1) == expect_count
    assert float(loss2) == float(loss1)
    # labels outside [0, c): ignored like F.nll_loss's ignore_index rows (not in the sum, not in the count,
    # zero gradient); torch's default ignore_index is -100
    y_ign = y.clone()
    y_ign[::7] = -100
    l2 = ops.log_softmax_nll_fwd(z.to(cuda), y_ign.to(cuda), m)
    l1 = ops.nll_loss_fwd(out, y_ign.to(cuda), m)
    assert float(l2[1]) == float(l1[0]) and int(l2[2]) == int(l1[1])
    counted = (y_ign >= 0) if mask is None else (mask & (y_ign >= 0))
    assert int(l1[1]) == int(counted.sum())
    dz_ign = ops.log_softmax_nll_bwd(out, y_ign.to(cuda), m, l1[1], gs.to(cuda))
    d_ign = ops.nll_loss_bwd(y_ign.to(cuda), m, l1[1], gs.to(cuda), n, c)
    assert float((dz_ign - ops.log_softmax_bwd(d_ign, out)).abs().max()) <= 1e-6
    if int(counted.sum()) > 0:
        zr = z.double().requires_grad_(True)
        ref = F.nll_loss(F.log_softmax(zr, dim=1)[sel], y_ign[sel])
        assert abs(float(l1[0]) - float(ref)) <= 1e-5 * max(1.0, abs(float(ref)))
        (ref * 0.5).backward()
        assert float((dz_ign.cpu().double() - zr.grad).abs().max()) <= 1e-6
        assert torch.count_nonzero(dz_ign[~counted.to(cuda)]) == 0
    else:
        assert float(l1[0]) == 0.0 and torch.count_nonzero(dz_ign) == 0
    y_bad = y.clone()
    y_bad[0] = c + 3                           # other labels outside the range are ignored the same way (torch raises)
    l2 = ops.log_softmax_nll_fwd(z.to(cuda), y_bad.to(cuda), m)
    l1 = ops.nll_loss_fwd(out, y_bad.to(cuda), m)
    assert float(l2[1]) == float(l1[0]) and int(l2[2]) == int(l1[1])
    assert int(l1[1]) == expect_count - (1 if (mask is None or bool(mask[0])) else 0)


def test_rowwise_kernels_on_views(cuda):
    """Rows inside a wider buffer: a 16-byte aligned view (leading dimension 32, 24 columns) takes the
    16-byte form, a view shifted by one float the element form; both must agree with torch."""
    from cagnet_amd import ops
    big = (_rand((500, 32), 21) * 3.0).to(cuda)
    g_big = _rand((500, 32), 22).to(cuda)
    for lo in (0, 1, 4):
        z, g = big[:, lo:lo + 24], g_big[:, lo:lo + 24]
        out = ops.log_softmax_fwd(z)
        ref = F.log_softmax(z.double(), dim=1)
        assert float((out.double() - ref).abs().max()) <= 1e-5 * max(1.0, float(ref.abs().max()))
        dz = ops.log_softmax_bwd(g, out)
        expect = g.double() - torch.exp(ref) * g.double().sum(dim=1, keepdim=True)
        scale = g.double().abs().sum(dim=1, keepdim=True)
        assert float(((dz.double() - expect).abs() / scale).max()) <= REL_TOL
    # ReLU on an unaligned flat range with a tail that is not a multiple of 4
    flat = _rand((1, 4099), 23).to(cuda).reshape(-1)
    for lo in (0, 1):
        v = flat[lo:lo + 4001]
        h = ops.relu_fwd(v.reshape(1, -1))
        assert torch.equal(h.reshape(-1), torch.relu(v))
        assert torch.equal(ops.relu_bwd(v.reshape(1, -1) * 2, h).reshape(-1), 2 * v * (v > 0))


def test_dense_vector_fallback_path(cuda):
    """The LDS-tiled vector kernel stays in the library for widths the matrix-core kernels do not
    cover (fo > 64); forcing it for a covered shape must give the same products."""
    from cagnet_amd import ops
    from cagnet_amd._lib import lib
    X, W, G = _rand((777, 300), 1), _rand((300, 24), 2), _rand((777, 24), 3)
    try:
        assert lib.cg_tune_set(b"dense_mfma", -1) == 0
        assert gemm_error(ops.dense_xw(X.to(cuda), W.to(cuda)), X, W) <= REL_TOL
        assert gemm_error(ops.dense_gwt(G.to(cuda), W.to(cuda)), G, W.t()) <= REL_TOL
        assert gemm_error(ops.dense_xtg(X.to(cuda), G.to(cuda)), X.t(), G) <= REL_TOL
    finally:
        lib.cg_tune_set(b"dense_mfma", 0)
    Wide = _rand((300, 100), 4)
    assert gemm_error(ops.dense_xw(X.to(cuda), Wide.to(cuda)), X, Wide) <= REL_TOL   # fo = 100 > 64
