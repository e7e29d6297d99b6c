"""The drop-in modules on the GPU: mixers against the oracle at module level, and the
reference's own correctness notion for this path — logits produced with the generation cache
equal the logits of a fresh parallel forward over the prefix (based/tests/test_generation.py)."""
import pytest
import torch
import torch.nn.functional as F

from conftest import rel_l2
from oracle import based_oracle as O

pytestmark = pytest.mark.gpu

# tolerances the reference's generation test accepts for bf16 (test_generation.py:106-115)
ATOL_BF16, RTOL_BF16 = 5e-2, 1e-2


def test_linear_attention_module_vs_oracle(dev):
    from based_amd.mixers import LinearAttention, TaylorExp

    torch.manual_seed(0)
    m = LinearAttention(d_model=256, feature_map=TaylorExp(input_dim=16), num_heads=4, head_dim=64,
                        layer_idx=0, device=dev, dtype=torch.bfloat16)
    for p in m.parameters():
        torch.nn.init.normal_(p, std=0.2)
    x = torch.randn(2, 96, 256, device=dev, dtype=torch.bfloat16)
    y = m(x)
    # oracle from the module's own projections (the GEMMs are torch on both sides)
    q = m.proj_q(x).view(2, 96, 4, 16).transpose(1, 2).float().cpu()
    k = m.proj_k(x).view(2, 96, 4, 16).transpose(1, 2).float().cpu()
    v = m.proj_v(x).view(2, 96, 4, 64).transpose(1, 2).float().cpu()
    yo = O.linear_attn_quadratic(q, k, v, eps=m.eps).transpose(1, 2).reshape(2, 96, 256)
    y_ref = F.linear(yo.to(torch.bfloat16).float(), m.out_proj.weight.float().cpu())
    assert y.shape == (2, 96, 256) and y.dtype == torch.bfloat16
    assert rel_l2(y.float(), y_ref) < 1.5e-2


def test_linear_attention_recurrent_forward_signature(dev):
    """recurrent_forward takes feature-mapped q, k (b, h, 1, 273) like the reference."""
    from based_amd.mixers import LinearAttention, TaylorExp

    torch.manual_seed(1)
    m = LinearAttention(d_model=128, feature_map=TaylorExp(input_dim=16), num_heads=2, head_dim=64,
                        layer_idx=0, device=dev, dtype=torch.bfloat16)
    kv, ks = m.allocate_inference_cache(3, 10)
    q = torch.randn(3, 2, 1, 16, device=dev, dtype=torch.bfloat16)
    k = torch.randn(3, 2, 1, 16, device=dev, dtype=torch.bfloat16)
    v = torch.randn(3, 2, 1, 64, device=dev, dtype=torch.bfloat16)
    kv_ref, ks_ref = kv.cpu().clone(), ks.cpu().clone()
    out = m.recurrent_forward(None, kv, ks, m.feature_map(q), m.feature_map(k), v)
    yo = O.linear_attn_step(kv_ref, ks_ref, q.float().cpu(), k.float().cpu(), v.float().cpu())
    y_ref = F.linear(yo.transpose(1, 2).reshape(3, 1, 128).to(torch.bfloat16).float(), m.out_proj.weight.float().cpu())
    assert rel_l2(out.float(), y_ref) < 1.5e-2
    assert rel_l2(kv, kv_ref) < 1e-5


@pytest.mark.parametrize("rotary", [0, 64])
def test_sliding_attention_module_vs_oracle(dev, rotary):
    from based_amd.mixers import SlidingAttention

    torch.manual_seed(2)
    m = SlidingAttention(embed_dim=256, num_heads=4, qkv_proj_bias=False, out_proj_bias=False, window_size=128,
                         layer_idx=0, rotary_emb_dim=rotary, device=dev, dtype=torch.bfloat16)
    for p in m.parameters():
        torch.nn.init.normal_(p, std=0.1)
    x = torch.randn(2, 200, 256, device=dev, dtype=torch.bfloat16)
    y = m(x)
    qkv = m.Wqkv(x).view(2, 200, 3, 4, 64)
    if rotary:
        qkv = m.rotary_emb(qkv)
    qkv = qkv.cpu()
    ctx = O.sliding_window_attn(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], w_left=64, scale=m.softmax_scale)
    y_ref = F.linear(ctx.reshape(2, 200, 256).float(), m.out_proj.weight.float().cpu())
    assert rel_l2(y.float(), y_ref) < 1.5e-2


def _small_stack(dev, rotary=0.0):
    from based_amd.stack import GPTLMHeadModel, based_360m_config

    cfg = based_360m_config(
        n_embd=256, n_head=4, n_layer=3, n_inner=512, vocab_size=1000, rotary_emb_fraction=rotary,
        alt_mixer={"_target_": "based.models.mixers.linear_attention.LinearAttention", "l_max": 2048,
                   "feature_map": {"_target_": "based.models.mixers.linear_attention.TaylorExp", "input_dim": 16},
                   "feature_dim": 16, "num_heads": 4},
        alt_mixer_layers=[1], alt_mixer_2_layers=[2])
    torch.manual_seed(3)
    model = GPTLMHeadModel(cfg, device=dev, dtype=torch.bfloat16)
    model.eval()
    return model


@pytest.mark.parametrize("prefill_size", [1, 128])
@pytest.mark.parametrize("rotary", [0.0, 1.0])
def test_generation_cached_equals_parallel(dev, prefill_size, rotary):
    """3-layer stack (BaseConv, LinearAttention, SlidingAttention), greedy generation with the
    cache vs a fresh parallel forward over every prefix."""
    model = _small_stack(dev, rotary)
    n_new = 64
    torch.manual_seed(0)
    input_ids = torch.randint(1, 1000, (4, prefill_size), dtype=torch.long, device=dev)
    out = model.generate(input_ids=input_ids, max_length=prefill_size + n_new, return_dict_in_generate=True,
                         output_scores=True, top_k=1)
    scores = torch.stack(out.scores, dim=1)
    seqs = out.sequences.clone()
    assert seqs.shape == (4, prefill_size + n_new)
    with torch.inference_mode():
        for i in range(n_new):
            ref = model(input_ids=seqs[:, : prefill_size + i]).logits[:, -1]
            # the reference's own assertion (based/tests/test_generation.py:169-173), on every logit
            assert torch.allclose(ref, scores[:, i], atol=ATOL_BF16, rtol=RTOL_BF16), f"position {i}"
            assert torch.equal(seqs[:, prefill_size + i], ref.argmax(dim=-1)), f"position {i}"


def test_graph_decode_equals_eager(dev):
    """Decoding through the recorded HIP graph (cg=True) against eager decoding of the same
    3-layer stack (BaseConv, LinearAttention, SlidingAttention with in-kernel rotary): same
    tokens, logits equal to bf16 noise.  The graph is replayed for several requests, with eager
    work and synchronisations in between, for another prompt length and for a smaller batch."""
    model = _small_stack(dev, rotary=1.0)
    n_new = 12
    for trial, (batch, prefill_size) in enumerate([(4, 33), (4, 33), (4, 70), (2, 5)]):
        print(f"graph decode trial {trial}: batch {batch} prefill {prefill_size}", flush=True)
        torch.manual_seed(trial)
        ids = torch.randint(1, 1000, (batch, prefill_size), dtype=torch.long, device=dev)
        eager = model.generate(input_ids=ids, max_length=prefill_size + n_new, return_dict_in_generate=True,
                               output_scores=True, top_k=1)
        torch.cuda.synchronize()
        graphed = model.generate(input_ids=ids, max_length=prefill_size + n_new, return_dict_in_generate=True,
                                 output_scores=True, top_k=1, cg=True)
        torch.cuda.synchronize()
        assert len(graphed.scores) == len(eager.scores) == n_new
        for i, (a, b_) in enumerate(zip(graphed.scores, eager.scores)):
            assert rel_l2(a.float(), b_.float()) < 1e-3, f"trial {trial} position {i}"
        assert torch.equal(graphed.sequences, eager.sequences)
    assert len(model._decoding_cache.callables) == 2  # one graph per batch size, reused across requests


def test_linear_attention_step_sees_weights_written_through_data(dev):
    """The single-token step projects through one stacked [q; k; v] matrix.  A write that bypasses
    the version counter (`weight.data.copy_`, what EMA swaps and some optimizers do) must reach
    it: the projections are views of the stacked storage, not copies."""
    from based_amd.generation import InferenceParams
    from based_amd.mixers import LinearAttention, TaylorExp

    torch.manual_seed(4)
    m = LinearAttention(d_model=256, feature_map=TaylorExp(input_dim=16), num_heads=4, head_dim=64,
                        layer_idx=0, device=dev, dtype=torch.bfloat16).eval()
    for p in m.parameters():
        torch.nn.init.normal_(p, std=0.2)

    def prefill_and_step(x, x1):
        params = InferenceParams(max_seqlen=64, max_batch_size=2)
        with torch.inference_mode():
            m(x, inference_params=params)
            params.seqlen_offset = x.shape[1]
            return m(x1, inference_params=params)

    x = torch.randn(2, 20, 256, device=dev, dtype=torch.bfloat16)
    x1 = torch.randn(2, 1, 256, device=dev, dtype=torch.bfloat16)
    before = prefill_and_step(x, x1)
    full = m(torch.cat([x, x1], dim=1))[:, -1:]
    assert rel_l2(before.float(), full.float()) < 1.5e-2
    new_q = torch.randn_like(m.proj_q.weight) * 0.2
    new_v = torch.randn_like(m.proj_v.weight) * 0.2
    v0 = m.proj_q.weight._version
    m.proj_q.weight.data.copy_(new_q)
    m.proj_v.weight.data.copy_(new_v)
    assert m.proj_q.weight._version == v0          # the write the cache key cannot see
    after = prefill_and_step(x, x1)
    full = m(torch.cat([x, x1], dim=1))[:, -1:]   # the parallel path reads the live weights
    assert rel_l2(after.float(), full.float()) < 1.5e-2
    assert rel_l2(after.float(), before.float()) > 0.1
    # a replaced tensor is noticed through its address
    m.proj_k.weight = torch.nn.Parameter(torch.randn_like(m.proj_k.weight) * 0.2)
    again = prefill_and_step(x, x1)
    assert rel_l2(again.float(), m(torch.cat([x, x1], dim=1))[:, -1:].float()) < 1.5e-2
    assert torch.equal(m.state_dict()["proj_q.weight"], new_q)
