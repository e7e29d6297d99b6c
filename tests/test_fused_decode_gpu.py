"""The single-token path of the stack with the projections as `ops.decode_linear` launches (norms and
SwiGLU gate folded into them, the embedding lookup into the first): it is the path taken, it stays
within the reference's bound of the oracle composition on every logit, it agrees with the general
path, and a recorded graph of it replays to the same logits."""
import pytest
import torch

from oracle import based_oracle as O

pytestmark = pytest.mark.gpu

ATOL, RTOL = 5e-2, 1e-2   # bf16 bound of based/tests/test_generation.py:106-115


def _cfg(**over):
    cfg = dict(
        n_embd=256, n_head=4, n_layer=4, n_inner=512, vocab_size=1000, pad_vocab_size_multiple=8, rms_norm=True,
        residual_in_fp32=True, activation_function="swiglu", mlp_type="base", layer_norm_epsilon=1e-5,
        mlp_fc1_bias=False, mlp_fc2_bias=False, qkv_proj_bias=True, out_proj_bias=True, max_position_embeddings=0,
        rotary_emb_fraction=1.0, scale_attn_weights=True, initializer_range=0.02,
        mixer={"_target_": "based.models.mixers.convolution.BaseConv", "l_max": 2048, "use_bias": True, "expand_proj": 4,
               "kernel_size": 3},
        alt_mixer={"_target_": "based.models.mixers.linear_attention.LinearAttention", "l_max": 2048,
                   "feature_map": {"_target_": "based.models.mixers.linear_attention.TaylorExp", "input_dim": 16},
                   "feature_dim": 16, "num_heads": 4},
        alt_mixer_layers=[1],
        alt_mixer_2={"_target_": "based.models.mixers.slide_attention.SlidingAttention", "window_size": 128,
                     "num_heads": 4, "causal": True},
        alt_mixer_2_layers=[2],
    )
    cfg.update(over)
    return cfg


def _build(cfg, dev, dtype=torch.bfloat16, seed=5):
    from based_amd.stack import GPTLMHeadModel, StackConfig

    torch.manual_seed(seed)
    model = GPTLMHeadModel(StackConfig(**cfg), device=dev, dtype=dtype).eval()
    with torch.no_grad():
        for name, p in model.named_parameters():
            if "norm" in name or "ln_f" in name:
                p.copy_(1.0 + 0.1 * torch.randn_like(p))
            elif name.endswith("bias"):
                p.copy_(0.05 * torch.randn_like(p))
    sd = {k: v.detach().float().cpu() for k, v in model.state_dict().items()}
    return model, sd


def _within(got, want, what, slack=1.0):
    got, want = got.float().cpu(), want.float().cpu()
    diff = (got - want).abs()
    bound = slack * (ATOL + RTOL * want.abs())
    assert float((diff - bound).max()) <= 0, f"{what}: max |diff| {float(diff.max()):.3e} exceeds the bound"


class _Calls:
    """Counts calls of the ops a decoding step goes through."""

    NAMES = ("decode_linear", "add_rms_norm", "swiglu", "linear_attn_step", "swa_step", "gated_conv_step")

    def __init__(self, monkeypatch):
        from based_amd import ops

        self.n = {k: 0 for k in self.NAMES}
        for name in self.NAMES:
            inner = getattr(ops, name)

            def counted(*a, _inner=inner, _name=name, **kw):
                self.n[_name] += 1
                return _inner(*a, **kw)

            monkeypatch.setattr(ops, name, counted)

    def reset(self):
        for k in self.n:
            self.n[k] = 0


@pytest.mark.parametrize("B", [1, 4, 9])
def test_fused_step_is_taken_and_matches_oracle_and_general_path(dev, monkeypatch, B):
    cfg = _cfg()
    model, sd = _build(cfg, dev)
    P, n_new = 70, 12
    torch.manual_seed(B)
    ids = torch.randint(1, 1000, (B, P), dtype=torch.long, device=dev)
    print(f"fused decode B={B}", flush=True)
    calls = _Calls(monkeypatch)
    fused = model.generate(input_ids=ids, max_length=P + n_new, return_dict_in_generate=True, output_scores=True, top_k=1)
    steps = len(fused.scores) - 1   # the first score is the prefill's
    n_layer = cfg["n_layer"]
    assert calls.n["decode_linear"] == steps * (4 * n_layer + 1)
    assert calls.n["linear_attn_step"] == steps and calls.n["swa_step"] == steps
    assert calls.n["gated_conv_step"] == 0   # the convolution step runs in the tail of in_proj
    # norms and gates of the steps ran inside the projections: what is counted here is the prefill's
    assert calls.n["add_rms_norm"] == 2 * n_layer + 1 and calls.n["swiglu"] == n_layer

    seqs = fused.sequences.cpu()
    for i, sc in enumerate(fused.scores):
        _within(sc, O.stack_forward(seqs[:, : P + i], sd, cfg)[:, -1], f"fused step {i} vs oracle")

    # the general path on the same tokens (teacher-forced, so that both see identical inputs)
    model.transformer.fused_decode = False
    calls.reset()
    general = model.generate(input_ids=ids, max_length=P + n_new, return_dict_in_generate=True, output_scores=True,
                             top_k=1, teacher_outputs=fused.sequences)
    assert calls.n["decode_linear"] == 0
    model.transformer.fused_decode = True
    for i, (a, b) in enumerate(zip(fused.scores, general.scores)):
        _within(a, b, f"fused vs general step {i}", slack=2.0)


def test_recorded_graph_of_the_fused_step(dev):
    cfg = _cfg()
    model, _ = _build(cfg, dev)
    B, P, n_new = 3, 40, 10
    torch.manual_seed(7)
    ids = torch.randint(1, 1000, (B, P), dtype=torch.long, device=dev)
    eager = model.generate(input_ids=ids, max_length=P + n_new, return_dict_in_generate=True, output_scores=True, top_k=1)
    for attempt in range(2):   # the second request replays the graph recorded by the first
        graph = model.generate(input_ids=ids, max_length=P + n_new, return_dict_in_generate=True, output_scores=True,
                               top_k=1, cg=True)
        torch.cuda.synchronize()
        assert torch.equal(graph.sequences, eager.sequences), f"request {attempt}"
        for i, (a, b) in enumerate(zip(graph.scores, eager.scores)):
            assert torch.equal(a, b), f"request {attempt}, step {i}"


def test_general_path_where_the_fused_one_does_not_apply(dev, monkeypatch):
    """fp32 weights, a batch beyond the kernel's row limit and a mixer without `decode_step`
    (ShortConvolution) all decode through the general path."""
    from based_amd import ops

    calls = _Calls(monkeypatch)
    cases = [
        (_cfg(alt_mixer_2_layers=[]), torch.float32, 2),
        (_cfg(), torch.bfloat16, ops.DECODE_LINEAR_MAX_ROWS + 1),
        (_cfg(mixer={"_target_": "based.models.mixers.convolution.ShortConvolution", "kernel_size": 3}), torch.bfloat16, 2),
    ]
    for cfg, dtype, B in cases:
        model, _ = _build(cfg, dev, dtype)
        ids = torch.randint(1, 1000, (B, 20), dtype=torch.long, device=dev)
        calls.reset()
        out = model.generate(input_ids=ids, max_length=24, return_dict_in_generate=True, output_scores=True, top_k=1)
        assert calls.n["decode_linear"] == 0 and calls.n["add_rms_norm"] > 0
        assert all(bool(torch.isfinite(s.float()).all()) for s in out.scores)


def test_transformer_alone_returns_the_normed_hidden_state(dev):
    """GPTModel.forward (no LM head) on the fused path equals the general path's output."""
    from based_amd.generation import InferenceParams

    cfg = _cfg()
    model, _ = _build(cfg, dev)
    body = model.transformer
    B, P = 2, 33
    ids = torch.randint(1, 1000, (B, P + 1), dtype=torch.long, device=dev)
    outs = []
    for fused in (True, False):
        body.fused_decode = fused
        ip = InferenceParams(max_seqlen=P + 8, max_batch_size=B)
        with torch.inference_mode():
            body(ids[:, :P], inference_params=ip)
            ip.seqlen_offset = P
            outs.append(body(ids[:, P:], inference_params=ip))
    body.fused_decode = True
    assert outs[0].shape == outs[1].shape == (B, 1, cfg["n_embd"])
    d = (outs[0].float() - outs[1].float()).abs()
    assert float(d.max()) <= 0.05 * float(outs[1].float().abs().max()) + 1e-3
