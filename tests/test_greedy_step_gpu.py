"""Greedy sampling step (`based_greedy_step`): the kernel against torch.argmax and the loop's own
bookkeeping (based/generation.py:64-70,190-204), and greedy decoding with the sampling recorded
inside the decode graph against eager decoding of the same model."""
import pytest
import torch

from based_amd import ops

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    return torch.device("cuda:0")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,V,Vpad", [(4, 50277, 50280), (1, 1000, 1000), (3, 37, 40), (5, 2049, 2049), (2, 8, 8)])
def test_greedy_step_matches_argmax_and_advances(dev, dtype, B, V, Vpad):
    g = torch.Generator().manual_seed(B * 131 + V)
    # coarse values: many exact ties, the first index must win
    logits = (torch.randint(-6, 7, (B, Vpad), generator=g).float() / 2).to(dtype).to(dev)
    logits[:, V:] = 100.0   # beyond vocab_size: must be ignored
    max_len = 12
    lengths = torch.tensor([(3 * b) % (max_len + 2) for b in range(B)], dtype=torch.int32, device=dev)
    seq = torch.full((B, max_len), -1, dtype=torch.long, device=dev)
    nxt = torch.full((B, 1), -7, dtype=torch.long, device=dev)
    pos = torch.full((B, 1), -7, dtype=torch.long, device=dev)
    before = lengths.clone()
    ops.greedy_step(logits, nxt, lengths, sequences=seq, position_ids=pos, vocab_size=V)
    torch.cuda.synchronize()
    want = logits[:, :V].float().argmax(dim=-1)
    # torch.argmax promises the first maximal index only on ties; check that independently
    mx = logits[:, :V].float().max(dim=-1).values
    first = torch.stack([(logits[b, :V].float() == mx[b]).nonzero()[0, 0] for b in range(B)])
    assert torch.equal(nxt[:, 0], first) and torch.equal(first, want)
    assert torch.equal(lengths, before + 1) and torch.equal(pos[:, 0], (before + 1).long())
    for b in range(B):
        col = int(before[b]) + 1
        row = seq[b].clone()
        if col < max_len:
            assert row[col] == first[b]
            row[col] = -1
        assert (row == -1).all()   # nothing else written, nothing out of range


def test_greedy_step_nan_is_largest_and_views(dev):
    """A NaN logit wins (the first one), as in torch.argmax; rows that are views with a stride, a
    misaligned base (scalar loads), no sequences and no position_ids are fine."""
    big = torch.randn(3, 600, device=dev)
    logits = big[:, 3:503]            # 12-byte offset: not 16-byte aligned
    logits[1, 77] = float("nan")
    logits[1, 300] = float("nan")
    lengths = torch.zeros(3, dtype=torch.int32, device=dev)
    nxt = torch.zeros(3, dtype=torch.long, device=dev)
    ops.greedy_step(logits, nxt, lengths)
    torch.cuda.synchronize()
    assert nxt[1] == 77
    assert nxt[0] == logits[0].argmax() and nxt[2] == logits[2].argmax()
    assert (lengths == 1).all()
    with pytest.raises(ValueError):
        ops.greedy_step(logits, nxt, lengths.long())
    with pytest.raises(ValueError):
        ops.greedy_step(logits, nxt, lengths, vocab_size=501)


def test_greedy_decoding_inside_the_graph_equals_eager(dev):
    """generate(cg=True) without scores records the sampling with the step: one graph replay per
    token.  Same tokens as eager decoding and as the graph path that returns scores, for several
    requests on one model (another prompt length, a smaller batch, a vocabulary bound), with eager
    work and synchronisations between the replays."""
    from based_amd.stack import GPTLMHeadModel, based_360m_config

    cfg = based_360m_config(
        n_embd=256, n_head=4, n_layer=3, n_inner=512, vocab_size=1000, rotary_emb_fraction=1.0,
        alt_mixer={"_target_": "based.models.mixers.linear_attention.LinearAttention", "l_max": 2048,
                   "feature_map": {"_target_": "based.models.mixers.linear_attention.TaylorExp", "input_dim": 16},
                   "feature_dim": 16, "num_heads": 4},
        alt_mixer_layers=[1], alt_mixer_2_layers=[2])
    torch.manual_seed(3)
    model = GPTLMHeadModel(cfg, device=dev, dtype=torch.bfloat16).eval()
    n_new = 12
    for trial, (batch, prefill_size, vocab) in enumerate([(4, 33, None), (4, 33, None), (4, 70, None), (2, 5, None),
                                                           (4, 20, 900), (4, 9, None)]):
        print(f"greedy graph decode trial {trial}: batch {batch} prefill {prefill_size} vocab {vocab}", flush=True)
        torch.manual_seed(100 + trial)
        ids = torch.randint(1, 900, (batch, prefill_size), dtype=torch.long, device=dev)
        kw = {} if vocab is None else {"vocab_size": vocab}
        eager = model.generate(input_ids=ids, max_length=prefill_size + n_new, top_k=1, **kw)
        torch.cuda.synchronize()
        fast = model.generate(input_ids=ids, max_length=prefill_size + n_new, top_k=1, cg=True, **kw)
        torch.cuda.synchronize()
        assert fast.shape == eager.shape == (batch, prefill_size + n_new)
        assert torch.equal(fast, eager), f"trial {trial}"
        if trial == 2:  # the scores-returning graph path on the same cache afterwards
            scored = model.generate(input_ids=ids, max_length=prefill_size + n_new, top_k=1, cg=True,
                                    return_dict_in_generate=True, output_scores=True)
            assert torch.equal(scored.sequences, eager) and len(scored.scores) == n_new
    # one prompt token, one new token
    ids = torch.randint(1, 900, (2, 1), dtype=torch.long, device=dev)
    assert torch.equal(model.generate(input_ids=ids, max_length=2, top_k=1, cg=True),
                       model.generate(input_ids=ids, max_length=2, top_k=1))
