"""Host-side logic that needs no GPU: module construction and parameter names, cache
shapes, config routing, sampling, and loud failure when tensors are not on a HIP device."""
import pytest
import torch

import based_amd
from based_amd import ops
from based_amd.generation import InferenceParams, sample
from based_amd.mixers import BaseConv, LinearAttention, SlidingAttention, TaylorExp
from based_amd.stack import GPTLMHeadModel, based_360m_config
from oracle import based_oracle as O


def test_linear_attention_parameters_and_cache():
    m = LinearAttention(d_model=1024, feature_map=TaylorExp(input_dim=16), feature_dim=16, num_heads=16, layer_idx=3)
    names = dict(m.named_parameters())
    assert set(names) == {"proj_q.weight", "proj_k.weight", "proj_v.weight", "out_proj.weight"}
    assert names["proj_q.weight"].shape == (256, 1024) and names["proj_v.weight"].shape == (1024, 1024)
    assert m.head_dim == 64 and m.expanded_size() == 273
    kv, ks = m.allocate_inference_cache(5, 100, dtype=torch.bfloat16)
    assert kv.shape == (5, 16, 1, 64, 273) and ks.shape == (5, 16, 1, 1, 273)
    assert kv.dtype == torch.float32  # state is carried in fp32


def test_taylor_module_matches_oracle():
    x = torch.randn(2, 3, 4, 16)
    fm = TaylorExp(input_dim=16)
    assert torch.allclose(fm(x), O.taylor_exp(x))
    assert torch.allclose(fm.raw_from_mapped(fm(x)), x)


def test_unsupported_feature_map_is_rejected():
    from based_amd.mixers import FeatureMap
    with pytest.raises(NotImplementedError):
        LinearAttention(d_model=64, feature_map=FeatureMap(input_dim=16), num_heads=4)
    with pytest.raises(NotImplementedError):
        LinearAttention(d_model=64, feature_map=TaylorExp(input_dim=8), feature_dim=8, num_heads=4)


def test_sliding_attention_parameters_and_cache():
    m = SlidingAttention(embed_dim=1024, num_heads=16, qkv_proj_bias=False, out_proj_bias=False, window_size=128, layer_idx=2)
    assert set(dict(m.named_parameters())) == {"Wqkv.weight", "out_proj.weight"}
    assert m.Wqkv.weight.shape == (3072, 1024) and m.window == (64, 0)
    assert m.allocate_inference_cache(3, 77).shape == (3, 77, 2, 16, 64)
    with pytest.raises(NotImplementedError):
        SlidingAttention(embed_dim=1024, num_heads=16, num_heads_kv=4)
    assert SlidingAttention(embed_dim=1024, num_heads=16, window_size=256).window == (128, 0)   # the released configs
    with pytest.raises(NotImplementedError):
        SlidingAttention(embed_dim=1024, num_heads=16, window_size=258)
    assert SlidingAttention(embed_dim=256, num_heads=16).head_dim == 16      # the reference's test models: plain kernel
    with pytest.raises(NotImplementedError):
        SlidingAttention(embed_dim=192, num_heads=16)                         # head dim 12


def test_cpu_tensors_fail_loudly():
    q = torch.zeros(1, 1, 1, 16)
    with pytest.raises(ValueError):
        ops.linear_attn_step(q, q, torch.zeros(1, 1, 1, 64), torch.zeros(1, 1, 1, 64, 273), torch.zeros(1, 1, 1, 1, 273))
    with pytest.raises(ValueError):
        ops.linear_attn_prefill(q, q, torch.zeros(1, 1, 1, 64))
    x = torch.zeros(1, 4, 2, 64, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ops.swa_prefill(x, x, x)
    with pytest.raises(ValueError):
        ops.swa_step(x[:, :1], x[:, :1], x[:, :1], torch.zeros(1, 8, 2, 2, 64, dtype=torch.bfloat16), 3)
    u = torch.zeros(2, 5, 32, dtype=torch.bfloat16)
    w = torch.zeros(16, 1, 3, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ops.gated_conv_prefill(u, w)
    with pytest.raises(ValueError):
        ops.gated_conv_step(u[:, :1], torch.zeros(2, 16, 3, dtype=torch.bfloat16), w)
    with pytest.raises(ValueError):
        ops.add_rms_norm(u, None, torch.ones(32, dtype=torch.bfloat16))
    with pytest.raises(ValueError):
        ops.swiglu(u)


def test_cpu_modules_fail_loudly():
    """The glue modules have no host-tensor path either: CPU tensors raise instead of taking
    some other implementation."""
    from based_amd.mixers.convolution import BaseConv, ShortConvolution
    from based_amd.stack import GatedMlp, RMSNorm

    x = torch.randn(2, 9, 32)
    with pytest.raises(ValueError):
        BaseConv(32, expand_proj=4)(x)
    with pytest.raises(ValueError):
        RMSNorm(32)(x)
    with pytest.raises(ValueError):
        GatedMlp(32, hidden_features=64)(x)
    with pytest.raises(ValueError):
        ShortConvolution(32, kernel_size=3)(x)
    # a LayerNorm stack (rms_norm: False, the reference's default) builds; its norms are torch modules
    ln_model = GPTLMHeadModel(based_360m_config(n_layer=1, vocab_size=64, rms_norm=False))
    assert isinstance(ln_model.transformer.ln_f, torch.nn.LayerNorm)
    assert "transformer.layers.0.norm1.bias" in ln_model.state_dict()


def test_stack_routing_and_state_dict_names():
    cfg = based_360m_config(n_layer=8, vocab_size=1000)
    model = GPTLMHeadModel(cfg)
    kinds = [type(l.mixer).__name__ for l in model.transformer.layers]
    assert kinds == ["BaseConv", "LinearAttention", "SlidingAttention", "BaseConv", "BaseConv", "BaseConv",
                     "LinearAttention", "SlidingAttention"]
    sd = model.state_dict()
    for key in ("transformer.layers.1.mixer.proj_q.weight", "transformer.layers.2.mixer.Wqkv.weight",
                "transformer.layers.0.mixer.in_proj.weight", "transformer.layers.0.mixer.conv.conv.weight",
                "transformer.layers.0.mlp.fc1.weight", "transformer.layers.0.norm1.weight",
                "transformer.embeddings.word_embeddings.weight", "transformer.ln_f.weight", "lm_head.weight"):
        assert key in sd, key
    assert sd["transformer.layers.0.mlp.fc1.weight"].shape == (4096, 1024)
    assert sd["transformer.layers.0.mlp.fc2.weight"].shape == (1024, 2048)
    assert sd["transformer.layers.0.mixer.conv.conv.weight"].shape == (2048, 1, 3)
    assert model.lm_head.weight is model.transformer.embeddings.word_embeddings.weight
    assert sd["lm_head.weight"].shape[0] % 8 == 0


def test_full_360m_parameter_count():
    model = GPTLMHeadModel(based_360m_config(), device="meta")
    n = sum(p.numel() for p in model.parameters())
    assert 355e6 < n < 370e6


def test_sampling():
    logits = torch.tensor([[0.1, 3.0, -1.0, 2.0], [5.0, 0.0, 0.0, 0.0]])
    assert sample(logits, top_k=1).tolist() == [1, 0]
    torch.manual_seed(0)
    for _ in range(20):
        t = sample(logits.clone(), top_k=2)
        assert t[0].item() in (1, 3) and t[1].item() in (0, 1, 2, 3)
    t = sample(logits.clone(), top_k=0, top_p=0.5)
    assert t[1].item() == 0


def test_inference_params_reset():
    ip = InferenceParams(max_seqlen=8, max_batch_size=2, lengths_per_sample=torch.ones(2, dtype=torch.int32))
    ip.seqlen_offset = 5
    ip.reset(16, 4)
    assert (ip.max_seqlen, ip.max_batch_size, ip.seqlen_offset) == (16, 4, 0)
    assert ip.lengths_per_sample.sum() == 0


def test_local_checkpoint_round_trip(tmp_path):
    """A checkpoint directory in the released layout (config.json + pytorch_model.bin with the
    training wrapper's "model." prefix and metric entries) loads into an identical model."""
    import json

    from based_amd.stack import GPTLMHeadModel, based_360m_config

    cfg = based_360m_config(n_embd=128, n_head=2, n_layer=3, n_inner=256, vocab_size=96,
                            alt_mixer={"_target_": "based.models.mixers.linear_attention.LinearAttention", "l_max": 64,
                                       "feature_map": {"_target_": "based.models.mixers.linear_attention.TaylorExp", "input_dim": 16},
                                       "feature_dim": 16, "num_heads": 2},
                            alt_mixer_layers=[1], alt_mixer_2_layers=[2])
    torch.manual_seed(1)
    src = GPTLMHeadModel(cfg)
    state = {"model." + k: v for k, v in src.state_dict().items()}
    state["train_metrics.num-tokens.count"] = torch.tensor(3)
    torch.save(state, tmp_path / "pytorch_model.bin")
    (tmp_path / "config.json").write_text(json.dumps(vars(cfg)))
    dst = GPTLMHeadModel.from_pretrained_local(str(tmp_path))
    a, b = src.state_dict(), dst.state_dict()
    assert a.keys() == b.keys()
    assert all(torch.equal(a[k], b[k]) for k in a)
    assert dst.lm_head.weight is dst.transformer.embeddings.word_embeddings.weight


def test_reference_config_defaults():
    """A config dictionary in the reference's format means here what it means there: missing keys
    take transformers' GPT2Config defaults and the getattr defaults of based/models/gpt.py."""
    from based_amd.stack import StackConfig

    c = StackConfig.from_reference_dict({"n_embd": 256, "n_head": 16, "rms_norm": True})
    assert (c.residual_in_fp32, c.mlp_fc1_bias, c.mlp_fc2_bias, c.qkv_proj_bias, c.out_proj_bias) == (False, True, True, True, True)
    assert c.vocab_size == 50257 and c.pad_vocab_size_multiple == 1 and c.n_layer == 12
    assert c.max_position_embeddings == 1024 and c.mlp_type == "base" and c.activation_function == "gelu_new"
    c = StackConfig.from_reference_dict({"max_position_embeddings": 0, "residual_in_fp32": True})
    assert c.max_position_embeddings == 0 and c.residual_in_fp32 is True


def test_old_layer_order_checkpoints_are_remapped():
    """Checkpoints written with the earlier order of the layers in a block (gpt.py:829-853):
    ln_0 -> layers.0.norm1, layers.l.norm1 -> layers.l.norm2, layers.l.norm2 -> layers.(l+1).norm1,
    last norm2 -> ln_f."""
    cfg = based_360m_config(n_embd=64, n_head=1, n_layer=3, n_inner=128, vocab_size=32,
                            alt_mixer_layers=[], alt_mixer_2_layers=[])
    torch.manual_seed(2)
    model = GPTLMHeadModel(cfg)
    sd = {k: v.clone() for k, v in model.state_dict().items()}
    norms = {}
    for name in ["transformer.ln_f"] + [f"transformer.layers.{l}.norm{j}" for l in range(3) for j in (1, 2)]:
        norms[name] = torch.randn(64)
        sd[name + ".weight"] = norms[name]
    # the same parameters filed under the old names
    old = dict(sd)
    old["transformer.ln_0.weight"] = old.pop("transformer.layers.0.norm1.weight")
    for l in range(3):
        old[f"transformer.layers.{l}.norm1.weight"] = sd[f"transformer.layers.{l}.norm2.weight"]
        nxt = f"transformer.layers.{l + 1}.norm1.weight" if l < 2 else "transformer.ln_f.weight"
        old[f"transformer.layers.{l}.norm2.weight"] = sd[nxt]
    del old["transformer.ln_f.weight"]
    model.load_state_dict(old)
    got = model.state_dict()
    for name, w in norms.items():
        assert torch.equal(got[name + ".weight"], w), name


def test_gated_mlp_variants_construct_like_the_reference():
    from based_amd.stack import GatedMlp

    alt = GatedMlp(256, hidden_features=2816, activation="geglu", mlp_type="alt", ff_mult=2)
    assert set(dict(alt.named_parameters())) == {"fc1.weight", "fc3.weight", "fc2.weight"}
    assert alt.fc1.weight.shape == (512, 256) and alt.fc2.weight.shape == (256, 512)   # int(2*256*2/3) -> 512
    base = GatedMlp(1024, hidden_features=2048)
    assert base.fc1.weight.shape == (4096, 1024) and base.fc2.weight.shape == (1024, 2048)
    with pytest.raises(NotImplementedError):
        GatedMlp(64, activation="gelu_new")
