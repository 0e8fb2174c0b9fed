"""cg_nll_loss_fwd_static, the entry point that allocates nothing, against cg_nll_loss_fwd.

Both run the same two kernels in the same order, so loss and count must be the same bits.  Two
calls in a row share the static device array; the second is smaller, so stale partial sums of the
first lie behind the ones it reads.
"""
import ctypes
from ctypes import c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu


def _call(fn, logp, y, mask, n, c):
    from cagnet_amd._lib import check
    loss = torch.full((), float("nan"), dtype=torch.float32, device=logp.device)
    count = torch.full((), -7, dtype=torch.int64, device=logp.device)
    st = fn(c_void_p(logp.data_ptr()), logp.stride(0), c_void_p(y.data_ptr()),
            c_void_p(mask.data_ptr()) if mask is not None else c_void_p(0), n, c, c_void_p(loss.data_ptr()),
            c_void_p(count.data_ptr()), c_void_p(torch.cuda.current_stream().cuda_stream))
    check(st, "nll")
    torch.cuda.synchronize()
    return loss.cpu(), count.cpu()


def _case(cuda, n, c, seed, frac):
    g = torch.Generator().manual_seed(seed)
    logp = torch.log_softmax(torch.randn(n, c, generator=g), dim=1).to(cuda)
    y = torch.randint(0, c, (n,), generator=g).to(cuda)
    mask = (torch.rand(n, generator=g) < frac).to(cuda) if frac is not None else None
    return logp, y, mask


def test_static_nll_matches_scratch_version_twice(cuda):
    from cagnet_amd._lib import lib
    from oracle import gcn_oracle as orc
    # the larger call first, the smaller second, then an empty mask and an empty input
    for n, c, seed, frac in ((300_001, 41, 1, 0.66), (1_000, 41, 2, 0.5), (5_000, 8, 3, 0.0), (777, 24, 4, None)):
        logp, y, mask = _case(cuda, n, c, seed, frac)
        want_loss, want_count = _call(lib.cg_nll_loss_fwd, logp, y, mask, n, c)
        got_loss, got_count = _call(lib.cg_nll_loss_fwd_static, logp, y, mask, n, c)
        assert int(got_count) == int(want_count) == (int(mask.sum()) if mask is not None else n)
        assert got_loss.view(torch.int32).item() == want_loss.view(torch.int32).item(), (n, c, got_loss, want_loss)
        ref = orc.masked_nll(logp.cpu().double(), y.cpu(), mask.cpu() if mask is not None else None)
        assert abs(float(got_loss) - float(ref)) <= 1e-5


def test_static_nll_rejects_sizes_beyond_its_array(cuda):
    from cagnet_amd._lib import lib
    logp, y, mask = _case(cuda, 16, 4, 5, None)
    loss = torch.zeros((), device=cuda)
    count = torch.zeros((), dtype=torch.int64, device=cuda)
    st = lib.cg_nll_loss_fwd_static(c_void_p(logp.data_ptr()), 4, c_void_p(y.data_ptr()), c_void_p(0), (1 << 24) + 1, 4,
                                    c_void_p(loss.data_ptr()), c_void_p(count.data_ptr()), c_void_p(0))
    assert st == 2  # CG_ERR_SIZE, before anything is launched
    assert b"static scratch" in lib.cg_last_error()
