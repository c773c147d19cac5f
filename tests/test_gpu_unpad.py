"""unpad_and_slice_tensor / gather_and_pad_tensor on one GPU against the layout oracle
(openrlhf/models/ring_attn_utils.py:103-182): index work, bit-exact."""
import pytest
import torch

from oracle import layout as olay

pytestmark = pytest.mark.gpu


def _dev():
    return torch.device("cuda:0")


def _mask(kind, batch, seqlen, g):
    m = torch.zeros(batch, seqlen, dtype=torch.long)
    for b in range(batch):
        if kind == "right":
            n = int(torch.randint(0, seqlen + 1, (1,), generator=g))
            m[b, :n] = 1
        elif kind == "left":
            n = int(torch.randint(0, seqlen + 1, (1,), generator=g))
            m[b, seqlen - n:] = 1
        elif kind == "both":
            lo = int(torch.randint(0, seqlen + 1, (1,), generator=g))
            hi = int(torch.randint(lo, seqlen + 1, (1,), generator=g))
            m[b, lo:hi] = 1
        elif kind == "holes":
            m[b] = (torch.rand(seqlen, generator=g) < 0.6).long()
        elif kind == "ones":
            m[b] = 1
    return m


@pytest.mark.parametrize("kind", ["right", "left", "both", "holes", "ones", "zeros"])
@pytest.mark.parametrize("batch,seqlen", [(1, 1), (2, 4), (3, 257), (7, 1024), (5, 1025), (4, 3000), (300, 37), (16, 4100)])
def test_unpad_matches_oracle(kind, batch, seqlen):
    from openrlhf_amd.models.ring_attn_utils import unpad_and_slice_tensor, unpad_indices

    g = torch.Generator().manual_seed(batch * 7919 + seqlen)
    mask = _mask(kind, batch, seqlen, g)
    seq = torch.randint(0, 151936, (batch, seqlen), generator=g)
    want = olay.unpad_and_slice_tensor(seq, mask)
    got = unpad_and_slice_tensor(seq.to(_dev()), mask.to(_dev()), None, return_cu_seqlens=True)
    names = ["sequences", "position_ids", "rolled_sequences", "ring_attn_pad_len", "indices", "cu_seqlens"]
    for name, w, gt in zip(names, want, got):
        if name == "ring_attn_pad_len":
            assert gt == 0 and w == 0
            continue
        assert tuple(gt.shape) == tuple(w.shape), (name, gt.shape, w.shape)
        assert torch.equal(gt.cpu().long(), w.long()), name
    assert got[0].dtype == seq.dtype and got[4].dtype == torch.int64
    assert torch.equal(unpad_indices(mask.to(_dev())).cpu(), want[4])


@pytest.mark.parametrize("mask_dtype", [torch.bool, torch.uint8, torch.int64, torch.float32])
def test_unpad_mask_dtypes(mask_dtype):
    from openrlhf_amd.models.ring_attn_utils import unpad_and_slice_tensor

    g = torch.Generator().manual_seed(5)
    mask = _mask("holes", 9, 1500, g)
    seq = torch.randint(0, 1000, (9, 1500), generator=g)
    want = olay.unpad_and_slice_tensor(seq, mask)
    got = unpad_and_slice_tensor(seq.to(_dev()), mask.to(mask_dtype).to(_dev()))
    for w, gt in zip(want[:3], got[:3]):
        assert torch.equal(gt.cpu(), w)
    assert torch.equal(got[4].cpu(), want[4])


def test_unpad_int32_and_strided_inputs():
    from openrlhf_amd.models.ring_attn_utils import unpad_and_slice_tensor

    g = torch.Generator().manual_seed(9)
    mask = _mask("both", 11, 700, g)
    seq = torch.randint(0, 1000, (11, 700), generator=g)
    want = olay.unpad_and_slice_tensor(seq, mask)
    seq_d = seq.to(torch.int32).t().contiguous().t().to(_dev())     # int32, column-major storage
    mask_d = mask.t().contiguous().t().to(_dev())
    got = unpad_and_slice_tensor(seq_d, mask_d, None)
    assert got[0].dtype == torch.int32 and got[2].dtype == torch.int32
    for w, gt in zip(want[:3], got[:3]):
        assert torch.equal(gt.cpu().long(), w)
    assert torch.equal(got[4].cpu(), want[4])


def test_unpad_reference_docstring_example():
    """The example in the reference's docstring (ring_attn_utils.py:112-118)."""
    from openrlhf_amd.models.ring_attn_utils import unpad_and_slice_tensor

    seq = torch.tensor([[1, 2, 3, 0], [4, 5, 0, 0]], device=_dev())
    mask = torch.tensor([[1, 1, 1, 0], [1, 1, 0, 0]], device=_dev())
    packed, pos, rolled, pad_len, indices = unpad_and_slice_tensor(seq, mask, None)
    assert packed.tolist() == [[1, 2, 3, 4, 5]]
    assert pos.tolist() == [[0, 1, 2, 0, 1]]
    assert rolled.tolist() == [[2, 3, 0, 5, 0]]
    assert indices.tolist() == [0, 1, 2, 4, 5] and pad_len == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.int64, torch.uint8])
@pytest.mark.parametrize("trailing", [(), (3,), (2, 5), (1,)])
def test_gather_and_pad_matches_oracle(dtype, trailing):
    from openrlhf_amd.models.ring_attn_utils import gather_and_pad_tensor

    g = torch.Generator().manual_seed(11)
    batch, seqlen = 6, 1300
    mask = _mask("holes", batch, seqlen, g)
    indices = torch.nonzero(mask.flatten()).flatten()
    n = indices.numel()
    vals = (torch.randn(1, n, *trailing, generator=g) * 50).to(dtype)
    want = olay.gather_and_pad_tensor(vals, indices, batch, seqlen)
    got = gather_and_pad_tensor(vals.to(_dev()), None, 0, indices.to(_dev()), batch, seqlen)
    # the reference pads the transposed [Ttot, 1, ...] tensor and squeezes the last axis
    # (ring_attn_utils.py:181): [1, Ttot] -> [B, T], [1, Ttot, 3] -> [B, T, 1, 3], [1, Ttot, 1] -> [B, T, 1]
    expect = {(): (batch, seqlen), (3,): (batch, seqlen, 1, 3), (2, 5): (batch, seqlen, 1, 2, 5), (1,): (batch, seqlen, 1)}
    assert tuple(got.shape) == tuple(want.shape) == expect[trailing]
    assert torch.equal(got.cpu(), want)


def test_gather_and_pad_round_trip_and_gradient():
    from openrlhf_amd.models.ring_attn_utils import gather_and_pad_tensor, unpad_and_slice_tensor

    g = torch.Generator().manual_seed(3)
    batch, seqlen = 5, 2100
    mask = _mask("both", batch, seqlen, g).to(_dev())
    seq = torch.randint(1, 1000, (batch, seqlen), generator=g).to(_dev())
    packed, _, _, _, indices = unpad_and_slice_tensor(seq, mask, None)
    back = gather_and_pad_tensor(packed, None, 0, indices, batch, seqlen)
    assert torch.equal(back, seq * mask)
    x = torch.randn(1, indices.numel(), device=_dev(), requires_grad=True)
    w = torch.randn(batch, seqlen, device=_dev())
    (gather_and_pad_tensor(x, None, 0, indices, batch, seqlen) * w).sum().backward()
    assert torch.equal(x.grad[0], w.reshape(-1)[indices])


def test_unpad_empty_and_errors():
    from openrlhf_amd.models.ring_attn_utils import gather_and_pad_tensor, unpad_and_slice_tensor

    seq = torch.zeros(3, 8, dtype=torch.long, device=_dev())
    packed, pos, rolled, pad_len, indices = unpad_and_slice_tensor(seq, torch.zeros_like(seq), None)
    assert packed.shape == (1, 0) and pos.shape == (1, 0) and rolled.shape == (1, 0) and indices.numel() == 0
    out = gather_and_pad_tensor(torch.zeros(1, 0, device=_dev()), None, 0, indices, 3, 8)
    assert out.shape == (3, 8) and not out.any()
    with pytest.raises(NotImplementedError):
        unpad_and_slice_tensor(seq, torch.ones_like(seq), object())
    with pytest.raises(ValueError):
        unpad_and_slice_tensor(seq, torch.ones(3, 7, dtype=torch.long, device=_dev()), None)


@pytest.mark.parametrize("kind", ["right", "left", "both", "holes", "full", "empty_rows"])
def test_tile_and_row_walks_agree(kind):
    """The C entry point with the per-tile counts (one workgroup per tile) and without them (one
    workgroup walks a row): the same outputs, bit for bit, on rows that span several tiles of
    ORLHF_UNPAD_TILE columns, and both equal the oracle."""
    from openrlhf_amd import _lib
    from openrlhf_amd._lib import call, ptr, stream_of

    g = torch.Generator().manual_seed(21)
    batch, seqlen = 7, 3 * _lib.UNPAD_TILE + 777
    if kind == "full":
        mask = torch.ones(batch, seqlen, dtype=torch.long)
    elif kind == "empty_rows":
        mask = _mask("holes", batch, seqlen, g)
        mask[1] = 0
        mask[5] = 0
    else:
        mask = _mask(kind, batch, seqlen, g)
    seq = torch.randint(0, 50000, (batch, seqlen), generator=g)
    want = olay.unpad_and_slice_tensor(seq, mask)
    d = _dev()
    seq_d, mask_d = seq.to(d), mask.to(torch.uint8).to(d)
    counts = torch.empty(batch, dtype=torch.int64, device=d)
    n_tiles = (seqlen + _lib.UNPAD_TILE - 1) // _lib.UNPAD_TILE
    tiles = torch.full((batch, n_tiles), -1, dtype=torch.int32, device=d)
    cu = torch.empty(batch + 1, dtype=torch.int64, device=d)
    st = stream_of(d)
    call("orlhf_mask_row_counts", ptr(mask_d), _lib.MASK_U8, batch, seqlen, ptr(counts), ptr(tiles), st)
    call("orlhf_cu_seqlens", ptr(counts), batch, ptr(cu), st)
    assert torch.equal(counts.cpu(), mask.sum(1))
    assert torch.equal(tiles.cpu().long(), torch.stack([mask[:, i * _lib.UNPAD_TILE:(i + 1) * _lib.UNPAD_TILE].sum(1) for i in range(n_tiles)], 1))
    total = int(cu[-1])
    outs = []
    for tile_counts in (tiles, None):
        out = torch.full((4, max(total, 1)), -7, dtype=torch.int64, device=d)
        call("orlhf_unpad_sequences", ptr(seq_d), ptr(mask_d), _lib.MASK_U8, batch, seqlen, ptr(cu), ptr(tile_counts), total,
             ptr(out[0]), ptr(out[1]), ptr(out[2]), ptr(out[3]), st)
        outs.append(out[:, :total].cpu())
    assert torch.equal(outs[0], outs[1])
    indices, packed, rolled, position = outs[0]
    assert torch.equal(packed, want[0][0]) and torch.equal(position, want[1][0]) and torch.equal(rolled, want[2][0])
    assert torch.equal(indices, want[4])
    # a capacity below the total: the slots past it are dropped, the others are unchanged
    if total > 100:
        cap = total - 37
        out = torch.full((4, total), -7, dtype=torch.int64, device=d)
        call("orlhf_unpad_sequences", ptr(seq_d), ptr(mask_d), _lib.MASK_U8, batch, seqlen, ptr(cu), ptr(tiles), cap,
             ptr(out[0]), ptr(out[1]), ptr(out[2]), ptr(out[3]), st)
        assert torch.equal(out[:, :cap].cpu(), outs[0][:, :cap]) and bool((out[:, cap:] == -7).all())
