"""artk_grpo_loss_static, the entry point that allocates nothing: called through the
C-ABI, its outputs must equal artk_grpo_loss's bit for bit (same kernels, scratch in a
static device array instead of a caller workspace), on two calls in a row, the second with
a smaller input; sizes beyond the maximum are rejected before any GPU work."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def make_inputs(T, S, seed, dev, with_ref):
    g = torch.Generator().manual_seed(seed)
    new = (-3.0 * torch.rand(T, generator=g)).to(dev)
    old = (new.cpu() + 0.3 * torch.randn(T, generator=g))
    old[torch.rand(T, generator=g) < 0.2] = float("nan")
    adv = torch.randn(T, generator=g)
    adv[torch.rand(T, generator=g) < 0.1] = 0.0
    mask = (torch.rand(T, generator=g) < 0.45).to(torch.uint8)
    w = torch.rand(T, generator=g) * 2
    ref = (new.cpu() + 0.1 * torch.randn(T, generator=g)).to(dev) if with_ref else None
    return new, old.to(dev), adv.to(dev), mask.to(dev), w.to(dev), ref, S


def both(lib, inp, beta, dev):
    """(scalars, coef) of artk_grpo_loss and of artk_grpo_loss_static on the same inputs."""
    from art_amd import _lib

    new, old, adv, mask, w, ref, S = inp
    T = new.numel()
    st = torch.cuda.current_stream(dev).cuda_stream
    refp = None if ref is None else ref.data_ptr()
    out = []
    for static in (False, True):
        scalars = torch.full((4,), float("nan"), dtype=torch.float32, device=dev)
        coef = torch.full((T,), float("nan"), dtype=torch.float32, device=dev)
        args = [new.data_ptr(), old.data_ptr(), adv.data_ptr(), mask.data_ptr(), w.data_ptr(), refp, 1, T, S,
                0.8, 1.25, beta, scalars.data_ptr(), coef.data_ptr()]
        if static:
            _lib.check(lib.artk_grpo_loss_static(*args, st))
        else:
            ws = torch.empty(lib.artk_grpo_loss_workspace_bytes(T), dtype=torch.uint8, device=dev)
            _lib.check(lib.artk_grpo_loss(*args, ws.data_ptr(), ws.numel(), st))
        torch.cuda.synchronize()
        out.append((scalars.cpu(), coef.cpu()))
    return out


def test_static_entry_matches_workspace_entry(artk_lib, gpu):
    from art_amd import _lib

    print("artk_grpo_loss_static: T=65536 then T=3072", flush=True)
    # a large call first, then a smaller one: the second must not see the first one's leftovers
    for T, S, seed, beta in ((65536, 8192, 1, 0.05), (3072, 1024, 2, 0.0)):
        inp = make_inputs(T, S, seed, gpu, beta > 0)
        (s_ws, c_ws), (s_st, c_st) = both(artk_lib, inp, beta, gpu)
        assert not torch.isnan(s_ws).any() and float(s_ws[3]) > 0
        assert torch.equal(s_ws.view(torch.int32), s_st.view(torch.int32)), (s_ws, s_st)
        assert torch.equal(c_ws.view(torch.int32), c_st.view(torch.int32))
    # beyond the static array: a clear error, nothing launched
    p = torch.empty(16, dtype=torch.float32, device=gpu).data_ptr()
    too_many = 262144 + 1024
    rc = artk_lib.artk_grpo_loss_static(p, p, p, p, p, None, 0, too_many, too_many, 0.8, 1.2, 0.0, p, p, None)
    assert rc == _lib.ERR_UNSUPPORTED_SHAPE
    assert b"at most 262144" in artk_lib.artk_last_error()
