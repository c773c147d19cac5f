"""orlhf_policy_loss_fwd_noalloc (partial sums in the library's built-in scratch array) against
orlhf_policy_loss_fwd (partial sums in a caller's workspace), through the C ABI: the same bits,
on two calls in a row, the second with a smaller input that leaves most of the scratch holding the
first call's contents."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _params(_lib, token_level, dual_clip, norm_value=None):
    p = _lib.PolicyParams()
    p.clip_eps_low, p.clip_eps_high, p.dual_clip = 0.2, 0.28, dual_clip
    p.policy_type, p.is_correction = _lib.POLICY_PPO, _lib.IS_TIS
    p.is_low, p.is_high = 0.9, 1.1
    p.token_level = 1 if token_level else 0
    keep = []
    p.norm = _lib.make_norm(2, norm_value, keep)
    return p


def _inputs(cuda, rows, cols, seed):
    g = torch.Generator().manual_seed(seed)
    old = -torch.rand(rows, cols, generator=g) * 3
    lp = old + torch.randn(rows, cols, generator=g) * 0.2
    roll = old + torch.randn(rows, cols, generator=g) * 0.05
    adv = torch.randn(rows, cols, generator=g)
    lens = torch.randint(1, cols + 1, (rows,), generator=g)
    lens[0] = cols
    mask = torch.arange(cols)[None, :] < lens[:, None]
    mask[rows // 2] = False  # an empty row
    return [t.to(cuda).contiguous() for t in (lp, old, adv, roll)], mask.to(cuda).contiguous()


def _both(lib, _lib, cuda, rows, cols, seed, token_level, norm_value):
    (lp, old, adv, roll), mask = _inputs(cuda, rows, cols, seed)
    params = _params(_lib, token_level, 3.0, norm_value)
    stream = _lib.stream_of(cuda)

    def outputs():
        return (torch.full((4,), -7.0, device=cuda), torch.full((rows,), -7.0, device=cuda),
                torch.full((rows, 2), -7.0, device=cuda))

    ws = torch.empty(lib.orlhf_token_workspace_bytes(rows, cols), dtype=torch.uint8, device=cuda)
    out_a, coef_a, aux_a = outputs()
    _lib.call("orlhf_policy_loss_fwd", lp.data_ptr(), old.data_ptr(), adv.data_ptr(), mask.data_ptr(), _lib.MASK_U8,
              roll.data_ptr(), rows, cols, None, ctypes.byref(params), ws.data_ptr(), out_a.data_ptr(),
              coef_a.data_ptr(), aux_a.data_ptr(), stream)
    out_b, coef_b, aux_b = outputs()
    _lib.call("orlhf_policy_loss_fwd_noalloc", lp.data_ptr(), old.data_ptr(), adv.data_ptr(), mask.data_ptr(),
              _lib.MASK_U8, roll.data_ptr(), rows, cols, None, ctypes.byref(params), out_b.data_ptr(),
              coef_b.data_ptr(), aux_b.data_ptr(), stream)
    torch.cuda.synchronize()
    assert torch.isfinite(out_a).all() and (out_a != -7.0).all()
    # bit-exact: the same kernels on the same inputs, only the partial sums live elsewhere
    assert torch.equal(out_a, out_b), (out_a, out_b)
    assert torch.equal(coef_a, coef_b) and torch.equal(aux_a, aux_b)
    return out_b


def test_no_alloc_entry_matches_workspace_entry_twice(lib, cuda):
    from openrlhf_amd import _lib

    first = _both(lib, _lib, cuda, 300, 5000, 1, True, None)         # 5 chunks per row
    second = _both(lib, _lib, cuda, 7, 300, 2, False, 5.0)           # smaller: stale partials stay beyond it
    third = _both(lib, _lib, cuda, 300, 5000, 1, True, None)         # and the first problem again
    assert torch.equal(first, third) and not torch.equal(first, second)


def test_no_alloc_entry_rejects_what_the_scratch_cannot_hold(lib, cuda):
    from openrlhf_amd import _lib

    rows, cols = 8192, 65536
    assert lib.orlhf_token_workspace_bytes(rows, cols) > (8 << 20)
    params = _params(_lib, True, 0.0)
    dummy = torch.zeros(8, device=cuda)
    with pytest.raises(_lib.KernelError, match="scratch"):
        _lib.call("orlhf_policy_loss_fwd_noalloc", dummy.data_ptr(), dummy.data_ptr(), dummy.data_ptr(), None,
                  _lib.MASK_NONE, None, rows, cols, None, ctypes.byref(params), dummy.data_ptr(), dummy.data_ptr(),
                  dummy.data_ptr(), _lib.stream_of(cuda))


def test_no_alloc_entry_replays_from_a_captured_graph(lib, cuda):
    """After one eager call on the device (which looks the scratch up) the entry may be captured: every
    replay, with eager calls on other shapes in between that leave their partial sums in the same
    scratch, gives the bits of the workspace entry on the inputs then in the captured buffers."""
    from openrlhf_amd import _lib

    rows, cols = 96, 4100
    _both(lib, _lib, cuda, 16, 900, 3, True, None)                   # the device's first call, eager
    (lp, old, adv, roll), mask = _inputs(cuda, rows, cols, 4)
    params = _params(_lib, True, 3.0)
    out, coef, aux = torch.zeros(4, device=cuda), torch.zeros(rows, device=cuda), torch.zeros(rows, 2, device=cuda)
    side = torch.cuda.Stream(device=cuda)
    side.wait_stream(torch.cuda.current_stream(cuda))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            _lib.call("orlhf_policy_loss_fwd_noalloc", lp.data_ptr(), old.data_ptr(), adv.data_ptr(), mask.data_ptr(),
                      _lib.MASK_U8, roll.data_ptr(), rows, cols, None, ctypes.byref(params), out.data_ptr(),
                      coef.data_ptr(), aux.data_ptr(), _lib.stream_of(cuda))
    torch.cuda.current_stream(cuda).wait_stream(side)
    ws = torch.empty(lib.orlhf_token_workspace_bytes(rows, cols), dtype=torch.uint8, device=cuda)
    for replay in range(3):
        (lp2, old2, adv2, roll2), _ = _inputs(cuda, rows, cols, 10 + replay)
        for dst, src in ((lp, lp2), (old, old2), (adv, adv2), (roll, roll2)):
            dst.copy_(src)
        out.fill_(-7.0)
        graph.replay()
        torch.cuda.synchronize()
        ref, rcoef, raux = torch.zeros(4, device=cuda), torch.zeros(rows, device=cuda), torch.zeros(rows, 2, device=cuda)
        _lib.call("orlhf_policy_loss_fwd", lp.data_ptr(), old.data_ptr(), adv.data_ptr(), mask.data_ptr(), _lib.MASK_U8,
                  roll.data_ptr(), rows, cols, None, ctypes.byref(params), ws.data_ptr(), ref.data_ptr(),
                  rcoef.data_ptr(), raux.data_ptr(), _lib.stream_of(cuda))
        torch.cuda.synchronize()
        assert torch.equal(out, ref) and torch.equal(coef, rcoef) and torch.equal(aux, raux), replay
        _both(lib, _lib, cuda, 300, 5000, replay, True, None)         # eager work through the same scratch
