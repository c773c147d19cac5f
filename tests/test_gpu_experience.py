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
