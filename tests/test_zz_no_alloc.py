"""slayer_li_bwd_static (the entry point that allocates nothing: its scratch is a buffer built into the
library) against slayer_li_bwd (scratch passed in by the caller), through the C ABI: two calls in a row
on the same GPU, the second on a smaller tensor, so the shared buffer still holds the first call's
contents.  Same kernels, so every output must agree bit for bit."""
import pytest
import torch

from lava_dl_amd.slayer import _native as N

pytestmark = pytest.mark.gpu


def both(shape, num_decays, seed):
    dev = torch.device('cuda:0')
    gen = torch.Generator().manual_seed(seed)
    grad_out = torch.randn(shape, generator=gen).to(dev)
    out = (torch.randn(shape, generator=gen) * 3).to(dev)
    decay = torch.randint(0, 4096, (num_decays,), generator=gen).float().to(dev)
    T = shape[-1]
    M = grad_out.numel() // T
    npb = M // shape[0]
    results = []
    for static in (False, True):
        grad_in = torch.full(shape, float('nan'), device=dev)
        grad_decay = torch.full((num_decays,), float('nan'), device=dev)
        stream = N.stream_handle()
        if static:
            code = N.lib().slayer_li_bwd_static(grad_in.data_ptr(), grad_decay.data_ptr(), grad_out.data_ptr(),
                                                out.data_ptr(), decay.data_ptr(), M, npb, num_decays, T, stream)
        else:
            ws = torch.empty(M + 64 * num_decays, device=dev)
            code = N.lib().slayer_li_bwd(grad_in.data_ptr(), grad_decay.data_ptr(), grad_out.data_ptr(),
                                         out.data_ptr(), decay.data_ptr(), ws.data_ptr(), M, npb, num_decays, T,
                                         stream)
        N.check(code)
        torch.cuda.synchronize()
        results.append((grad_in.cpu(), grad_decay.cpu()))
    return results


def test_static_scratch_entry_point_matches_the_workspace_one_on_two_calls_in_a_row():
    for shape, num_decays, seed in (((8, 16, 12, 12, 300), 16, 1), ((4, 16, 200), 1, 2), ((2, 6, 40), 6, 3)):
        print('li_bwd_static case', shape, num_decays, seed, flush=True)
        (gi_ws, gd_ws), (gi_st, gd_st) = both(shape, num_decays, seed)
        assert not torch.isnan(gi_st).any() and not torch.isnan(gd_st).any()
        assert torch.equal(gi_ws, gi_st), shape
        assert torch.equal(gd_ws, gd_st), shape


def test_static_scratch_entry_point_without_parameter_gradient_and_size_limit():
    dev = torch.device('cuda:0')
    gen = torch.Generator().manual_seed(7)
    shape = (3, 5, 64)
    grad_out = torch.randn(shape, generator=gen).to(dev)
    out = torch.randn(shape, generator=gen).to(dev)
    decay = torch.tensor([100.0], device=dev)
    a = torch.empty(shape, device=dev)
    b = torch.empty(shape, device=dev)
    st = N.stream_handle()
    N.check(N.lib().slayer_li_bwd_static(a.data_ptr(), None, grad_out.data_ptr(), out.data_ptr(), decay.data_ptr(),
                                         15, 5, 1, 64, st))
    N.check(N.lib().slayer_li_bwd(b.data_ptr(), None, grad_out.data_ptr(), out.data_ptr(), decay.data_ptr(), None,
                                  15, 5, 1, 64, st))
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    too_many = (1 << 20) + 1
    assert N.lib().slayer_li_bwd_static(a.data_ptr(), a.data_ptr(), a.data_ptr(), a.data_ptr(), a.data_ptr(),
                                        too_many, too_many, 1, 4, st) == -4
