"""The Experience container and its batch helpers
(openrlhf/trainer/ppo_utils/experience.py:29-283): split / un-pad / re-batch / concatenate /
balance against known answers and the layout oracle, on GPU tensors and on the controller's CPU
tensors (padding runs through the row kernels either way)."""
from types import SimpleNamespace

import pytest
import torch

from oracle import layout as olay

pytestmark = pytest.mark.gpu


def _batch(dev, lens=(7, 4, 9), prompt=3, t=10, seed=0):
    from openrlhf_amd.trainer.ppo_utils.experience import Experience

    g = torch.Generator().manual_seed(seed)
    b = len(lens)
    att = (torch.arange(t)[None, :] < torch.tensor(lens)[:, None]).long()
    seqs = torch.randint(1, 1000, (b, t), generator=g) * att
    amask = att[:, 1:].bool().clone()
    amask[:, : prompt - 1] = False
    lp = torch.randn(b, t - 1, generator=g) * amask
    return Experience(
        sequences=seqs.to(dev), attention_mask=att.to(dev), action_mask=amask.to(dev), action_log_probs=lp.to(dev),
        values=(torch.randn(b, t - 1, generator=g) * amask).to(dev), rewards=torch.randn(b, generator=g).to(dev),
        total_length=torch.tensor(lens).to(dev), response_length=(torch.tensor(lens) - prompt).to(dev),
        prompts=[f"p{i}" for i in range(b)], labels=[f"l{i}" for i in range(b)],
        info={"reward": torch.randn(b, generator=g).to(dev), "tag": [f"t{i}" for i in range(b)]},
    )


@pytest.mark.parametrize("where", ["cuda", "cpu"])
def test_split_unpad_rebatch_round_trip(cuda, where):
    from openrlhf_amd.trainer.ppo_utils.experience import (
        Experience, make_experience_batch, remove_padding_in_sequences, split_experience_batch)

    dev = cuda if where == "cuda" else torch.device("cpu")
    lens = (7, 4, 9)
    exp = _batch(dev, lens)
    items = split_experience_batch(exp)
    assert len(items) == 3 and exp.index is None
    assert items[1].sequences.shape == (10,) and items[1].prompts == ["p1"] and items[1].info["tag"] == "t1"
    items = remove_padding_in_sequences(items)
    for row, (it, n) in enumerate(zip(items, lens)):
        assert it.sequences.shape == (n,) and it.attention_mask.shape == (n,)
        assert it.action_mask.shape == (n - 1,) and it.values.shape == (n - 1,)  # A = T - 1 columns lose the same tail
        assert it.attention_mask.all()
        assert n == olay.unpadded_length(exp.attention_mask[row].cpu())
    again = make_experience_batch(items)
    assert again.sequences.device.type == dev.type
    # the widest sample has 9 tokens: the re-batched block is [3, 9], right-padded with zeros
    assert again.sequences.shape == (3, 9) and torch.equal(again.sequences, exp.sequences[:, :9])
    assert torch.equal(again.action_log_probs, exp.action_log_probs[:, :8])
    assert again.action_mask.dtype == torch.bool and torch.equal(again.action_mask, exp.action_mask[:, :8])
    assert torch.equal(again.rewards, exp.rewards) and torch.equal(again.total_length, exp.total_length)
    assert again.prompts == exp.prompts and again.info["tag"] == ["t0", "t1", "t2"]
    # tensor-valued info entries stay a list of per-sample 0-dim tensors, as in the reference
    assert isinstance(again.info["reward"], list) and torch.equal(torch.stack(again.info["reward"]), exp.info["reward"])
    want = olay.zero_pad_sequences([it.values.cpu() for it in items], "right", 0, stack=True)
    assert torch.equal(again.values.cpu(), want)
    with pytest.raises(ValueError):
        make_experience_batch([])
    assert Experience.is_step_tensor_field("kl") and Experience.is_episode_tensor_field("scores")
    assert not Experience.is_step_tensor_field("rewards") and not Experience.is_episode_tensor_field("prompts")


def test_all_zero_attention_mask_keeps_everything(cuda):
    from openrlhf_amd.trainer.ppo_utils.experience import remove_padding_in_sequences, split_experience_batch

    exp = _batch(cuda, (5, 10))
    exp.attention_mask[0] = 0  # flip(0).argmax() of zeros is 0: the reference cuts nothing
    items = remove_padding_in_sequences(split_experience_batch(exp))
    assert items[0].sequences.shape == (10,) and items[1].sequences.shape == (10,)


def test_concat_pads_token_ids_with_the_pad_token(cuda):
    from openrlhf_amd.trainer.ppo_utils.experience import Experience

    a, b = _batch(cuda, (7, 4), t=8, seed=1), _batch(cuda, (9, 9, 2), t=10, seed=2)
    cat = Experience.concat_experiences([a, b], pad_token_id=151643)
    assert cat.sequences.shape == (5, 10) and cat.action_log_probs.shape == (5, 9)
    assert torch.equal(cat.sequences[:2, :8], a.sequences) and (cat.sequences[:2, 8:] == 151643).all()
    assert torch.equal(cat.sequences[2:], b.sequences)
    assert (cat.attention_mask[:2, 8:] == 0).all() and (cat.action_log_probs[:2, 7:] == 0).all()
    # per-episode [B] tensors go through the same last-dimension padding in the reference, so
    # batches of different sizes are padded to the larger one before they are concatenated
    want = olay.zero_pad_sequences([a.rewards.cpu(), b.rewards.cpu()], "right", 0)
    assert want.shape == (6,) and torch.equal(cat.rewards.cpu(), want)
    assert cat.prompts == a.prompts + b.prompts and cat.info["tag"] == a.info["tag"] + b.info["tag"]
    same = Experience.concat_experiences([a, _batch(cuda, (3, 8), t=8, seed=5)], pad_token_id=0)
    assert same.rewards.shape == (4,) and torch.equal(same.rewards[:2], a.rewards)
    assert Experience.concat_experiences([], 0).sequences is None


def test_balance_interleaves_long_and_short(cuda):
    """The example of the reference's docstring: lengths 8..1 over 2 ranks -> [8,1,6,3], [7,2,5,4]."""
    from openrlhf_amd.trainer.ppo_utils.experience import Experience, balance_experiences

    def single(n):
        att = torch.ones(1, n, dtype=torch.long, device=cuda)
        return Experience(sequences=att.clone(), attention_mask=att, action_mask=att[:, 1:].bool(),
                          total_length=torch.tensor([n], device=cuda))

    exps = [single(n) for n in (3, 8, 1, 6, 2, 7, 5, 4)]
    args = SimpleNamespace(actor=SimpleNamespace(num_nodes=1, num_gpus_per_node=2),
                           ds=SimpleNamespace(ring_attn_size=1, tensor_parallel_size=1))
    out = balance_experiences(exps, args)
    assert [e.total_length.tolist() for e in out] == [[8, 1, 6, 3], [7, 2, 5, 4]]
    assert out[0].sequences.shape == (4, 8) and out[0].attention_mask.sum(1).tolist() == [8, 1, 6, 3]
    odd = balance_experiences(exps[:5], args)  # 3, 8, 1, 6, 2 -> chunks [8,6] [3,2] [1]
    assert sorted(sum((e.total_length.tolist() for e in odd), [])) == [1, 2, 3, 6, 8]


def test_packed_fields_of_an_experience(cuda):
    from openrlhf_amd.models.loss import PolicyLoss
    from openrlhf_amd.trainer.ppo_utils.experience import PackedSteps

    exp = _batch(cuda, (7, 4, 9, 10))
    ps = exp.packed()
    assert set(ps.fields) == {"action_mask", "action_log_probs", "values"}  # the [B, A] fields that are set
    ref = PackedSteps.from_padded(dict(action_log_probs=exp.action_log_probs), exp.action_mask)
    assert torch.equal(ps["action_log_probs"], ref["action_log_probs"]) and torch.equal(ps.cu_seqlens, ref.cu_seqlens)
    old = exp.action_log_probs + 0.01
    adv = exp.values
    padded = PolicyLoss()(exp.action_log_probs, old, adv, action_mask=exp.action_mask)[0]
    po = PackedSteps.from_padded(dict(old=old, adv=adv), exp.action_mask)
    packed = PolicyLoss()(ps["action_log_probs"], po["old"], po["adv"], action_mask=ps["action_mask"],
                          cu_seqlens=ps.cu_seqlens, max_seqlen=ps.max_seqlen)[0]
    assert abs(padded.item() - packed.item()) <= 1e-6


def _ragged_batch(dev, seed=3, b=9, t=41):
    """Right-padded rows of every length from 1 to t, one row without padding, one all-zero mask."""
    from openrlhf_amd.trainer.ppo_utils.experience import Experience

    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(1, t + 1, (b,), generator=g)
    lens[0], lens[1] = t, 0
    att = (torch.arange(t)[None, :] < lens[:, None]).long()
    a = t - 1
    amask = att[:, 1:].bool().clone()
    amask[:, :2] = False
    amask[3, 5:9] = False  # a hole inside a row stays inside its extent
    mk = lambda: torch.randn(b, a, generator=g)
    return Experience(
        sequences=torch.randint(1, 1000, (b, t), generator=g).to(dev), attention_mask=att.to(dev),
        action_mask=amask.to(dev), action_log_probs=mk().to(dev), base_action_log_probs=mk().to(dev),
        values=mk().to(dev), kl=mk().to(torch.bfloat16).to(dev), rewards=torch.randn(b, generator=g).to(dev),
        total_length=lens.to(dev), prompts=[f"p{i}" for i in range(b)], labels=[f"l{i}" for i in range(b)],
        info={"tag": [f"t{i}" for i in range(b)], "score": torch.arange(b).float().to(dev)},
    ), lens


def _reference_hops(exp, rows=None):
    """What the reference's hops build from the batch: split, cut the padding, re-batch (the
    mirrors of experience.py:164-247, themselves checked against the layout oracle above)."""
    import copy

    from openrlhf_amd.trainer.ppo_utils.experience import (
        make_experience_batch, remove_padding_in_sequences, split_experience_batch)

    items = remove_padding_in_sequences(split_experience_batch(copy.copy(exp)))
    if rows is not None:
        items = [items[r] for r in rows]
    return make_experience_batch(items), items


def test_packed_experience_equals_the_reference_hops(cuda):
    from openrlhf_amd.trainer.ppo_utils.experience import STEP_FIELDS, PackedExperience

    exp, lens = _ragged_batch(cuda)
    want, items = _reference_hops(exp)
    pe = PackedExperience.from_experience(exp)
    assert len(pe) == 9
    # every flat field is the concatenation of what remove_padding_in_sequences keeps of each sample
    for name in ("sequences", "attention_mask", "action_mask", "action_log_probs", "values", "kl"):
        cat = torch.cat([getattr(it, name) for it in items])
        assert pe.steps[name].dtype == cat.dtype and torch.equal(pe.steps[name], cat), name
    keep = [olay.unpadded_length(exp.attention_mask[r].cpu()) for r in range(9)]
    assert pe.cu[41].tolist() == [0] + torch.tensor(keep).cumsum(0).tolist()
    got = pe.to_experience()
    # straight against the layout oracle's restatement of the three hops
    for name in ("sequences", "attention_mask", "action_mask", "action_log_probs", "base_action_log_probs", "values", "kl"):
        ref, kept = olay.unpad_and_rebatch(getattr(exp, name).cpu(), exp.attention_mask.cpu())
        assert torch.equal(getattr(got, name).cpu(), ref), name
        w_ = getattr(exp, name).shape[1]
        assert (pe.cu[w_][1:] - pe.cu[w_][:-1]).tolist() == kept, name
    for name in STEP_FIELDS:
        w, g_ = getattr(want, name), getattr(got, name)
        assert (w is None) == (g_ is None), name
        if w is not None:
            assert w.shape == g_.shape and w.dtype == g_.dtype and torch.equal(w, g_), name
    assert torch.equal(got.rewards, exp.rewards) and got.prompts == exp.prompts and got.info["tag"] == exp.info["tag"]
    # a known padded width saves the read-back
    assert torch.equal(pe.to_experience(widths={41: 41, 40: 40}).values, want.values)


def test_packed_experience_select_and_concat(cuda):
    from openrlhf_amd.trainer.ppo_utils.experience import PackedExperience

    exp, _ = _ragged_batch(cuda, seed=5)
    pe = PackedExperience.from_experience(exp)
    rows = [4, 0, 4, 8, 1, -2]
    sub = pe.select(rows)
    want, _ = _reference_hops(exp, [r % 9 for r in rows])
    got = sub.to_experience()
    for name in ("sequences", "attention_mask", "action_mask", "action_log_probs", "base_action_log_probs", "values", "kl"):
        assert torch.equal(getattr(got, name), getattr(want, name)), name
    assert torch.equal(got.rewards, exp.rewards[[4, 0, 4, 8, 1, 7]]) and got.prompts == ["p4", "p0", "p4", "p8", "p1", "p7"]
    assert got.info["tag"] == ["t4", "t0", "t4", "t8", "t1", "t7"] and torch.equal(got.info["score"], exp.info["score"][[4, 0, 4, 8, 1, 7]])
    with pytest.raises(IndexError):
        pe.select([9])
    assert len(pe.select([])) == 0 and pe.select([]).steps["values"].numel() == 0
    # two halves joined again are the whole
    both = PackedExperience.concat([pe.select(range(0, 4)), pe.select(range(4, 9))])
    for name, flat in pe.steps.items():
        assert torch.equal(both.steps[name], flat), name
    assert torch.equal(both.cu[40], pe.cu[40]) and both.meta["prompts"] == exp.prompts
    assert torch.equal(both.episode["rewards"], exp.rewards)


def test_packed_experience_feeds_the_per_token_kernels(cuda):
    """Advantages computed on the packed fields and stored back equal the padded computation on the
    columns the samples keep."""
    from openrlhf_amd.trainer.ppo_utils.experience import PackedExperience
    from openrlhf_amd.trainer.ppo_utils.experience_maker import get_advantages_and_returns

    exp, _ = _ragged_batch(cuda, seed=7)
    exp.values = exp.values * exp.action_mask
    rewards = exp.action_log_probs * exp.action_mask
    adv_p, ret_p = get_advantages_and_returns(exp.values, rewards, exp.action_mask, 0.99, 0.95)
    pe = PackedExperience.from_experience(exp)
    pe.set_step("rewards_t", pe.steps["action_log_probs"] * pe.steps["action_mask"])
    ps = pe.actions()
    adv, ret = get_advantages_and_returns(ps["values"], ps["rewards_t"], ps["action_mask"], 0.99, 0.95,
                                          cu_seqlens=ps.cu_seqlens, max_seqlen=ps.max_seqlen, row_order=ps.longest_first)
    pe.set_step("advantages", adv)
    pe.set_step("returns", ret)
    got = pe.to_experience()
    width = got.advantages.shape[1]
    keep = (torch.arange(width, device=cuda)[None, :] < (pe.cu[40][1:] - pe.cu[40][:-1])[:, None])
    # behind a row's last attended token the padded scan sees zeros only, so the kept columns agree
    assert torch.allclose(got.advantages, adv_p[:, :width] * keep, rtol=1e-6, atol=1e-6)
    assert torch.allclose(got.returns, ret_p[:, :width] * keep, rtol=1e-6, atol=1e-6)
    with pytest.raises(ValueError):
        pe.set_step("bad", adv[:-1])
