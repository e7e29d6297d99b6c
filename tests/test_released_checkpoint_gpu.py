"""A checkpoint in the layout of the released Based models, loaded and run on the GPU.

The directory holds `config.json` with the model section of
train/configs/experiment/reference/based-360m.yaml:49-117 as written (window_size 256, rotary over
the whole head, parallel_implementation "fla_parallel", explicit max_position_embeddings 0, the
yaml's `kernel_sizes` key included), shrunk only in width, depth and vocabulary so the CPU oracle
finishes in seconds, and `pytorch_model.bin` with the reference's parameter names under the
"model." prefix that from_pretrained_hf strips (gpt.py:446-459).  The weights are drawn here,
tensor by tensor, not by this package's initialiser: the names and shapes are the contract.
The loaded model's prefill logits and every cached decode step are held against the oracle
composition at the reference's own bf16 bound on every logit (tests/test_generation.py:106-115).
"""
import json

import pytest
import torch

from oracle import based_oracle as O

pytestmark = pytest.mark.gpu

N_EMBD, N_HEAD, N_LAYER, VOCAB = 256, 4, 4, 1000


def released_config(N_EMBD=N_EMBD, N_HEAD=N_HEAD, N_LAYER=N_LAYER):
    return {
        "alt_mixer_layers": [1], "alt_mixer_2_layers": [2],
        "mixer": {"_target_": "based.models.mixers.convolution.BaseConv", "l_max": 2048, "use_bias": True,
                  "expand_proj": 4, "kernel_sizes": 3},
        "alt_mixer": {"_target_": "based.models.mixers.linear_attention.LinearAttention", "l_max": 2048,
                      "feature_map": {"_target_": "based.models.mixers.linear_attention.TaylorExp", "input_dim": 16},
                      "feature_dim": 16, "num_heads": N_HEAD, "parallel_implementation": "fla_parallel"},
        "alt_mixer_2": {"_target_": "based.models.mixers.slide_attention.SlidingAttention", "window_size": 256,
                        "num_heads": N_HEAD, "causal": True},
        "n_embd": N_EMBD, "special_initializer": True, "n_head": N_HEAD, "n_layer": N_LAYER,
        "_target_": "based.models.gpt.GPT2MixerConfig", "rms_norm": True, "fused_mlp": False, "attn_pdrop": 0,
        "embd_pdrop": 0, "n_positions": 2048, "resid_pdrop": 0, "mlp_fc1_bias": False, "mlp_fc2_bias": False,
        "fused_bias_fc": True, "out_proj_bias": False, "qkv_proj_bias": False, "use_flash_attn": True,
        "residual_in_fp32": True, "activation_function": "swiglu", "rotary_emb_fraction": 1,
        "fused_dropout_add_ln": True, "max_position_embeddings": 0, "pad_vocab_size_multiple": 8,
        "reorder_and_upcast_attn": False, "scale_attn_by_inverse_layer_idx": False, "n_inner": 2 * N_EMBD,
        "vocab_size": VOCAB,
    }


def released_state_dict(cfg, seed=11):
    """The reference's parameter names and shapes for this configuration (gpt.py:64-96 routing;
    convolution.py:186-193, linear_attention.py:103-106, slide_attention.py:527-547, mlp.py:118-139)."""
    g = torch.Generator().manual_seed(seed)
    d, inner = cfg["n_embd"], cfg["n_inner"]
    mat = lambda *shape: (0.02 * torch.randn(*shape, generator=g)).bfloat16()
    vec = lambda n: (0.02 * torch.randn(n, generator=g)).bfloat16()
    gain = lambda n: (1.0 + 0.1 * torch.randn(n, generator=g)).bfloat16()
    sd = {"transformer.embeddings.word_embeddings.weight": mat(VOCAB, d)}   # vocab 1000 is a multiple of 8
    for i in range(cfg["n_layer"]):
        p = f"transformer.layers.{i}."
        sd[p + "norm1.weight"], sd[p + "norm2.weight"] = gain(d), gain(d)
        if i in cfg["alt_mixer_2_layers"]:
            sd[p + "mixer.Wqkv.weight"], sd[p + "mixer.out_proj.weight"] = mat(3 * d, d), mat(d, d)
        elif i in cfg["alt_mixer_layers"]:
            h = cfg["alt_mixer"]["num_heads"]
            # q, k entries of standard deviation 2.56 at any width (8 x 0.02 x sqrt(256)): scores of a few units
            qk_gain = 8 * (256 / d) ** 0.5
            sd[p + "mixer.proj_q.weight"] = (qk_gain * mat(16 * h, d).float()).bfloat16()
            sd[p + "mixer.proj_k.weight"] = (qk_gain * mat(16 * h, d).float()).bfloat16()
            sd[p + "mixer.proj_v.weight"], sd[p + "mixer.out_proj.weight"] = mat(d, d), mat(d, d)
        else:
            d_inner = 4 * d // 2
            sd[p + "mixer.in_proj.weight"], sd[p + "mixer.in_proj.bias"] = mat(4 * d, d), vec(4 * d)
            sd[p + "mixer.out_proj.weight"], sd[p + "mixer.out_proj.bias"] = mat(d, d_inner), vec(d)
            sd[p + "mixer.conv.conv.weight"] = (0.3 * torch.randn(d_inner, 1, 3, generator=g)).bfloat16()
        sd[p + "mlp.fc1.weight"], sd[p + "mlp.fc2.weight"] = mat(2 * inner, d), mat(d, inner)
    sd["transformer.ln_f.weight"] = gain(d)
    sd["lm_head.weight"] = sd["transformer.embeddings.word_embeddings.weight"]   # tied
    return sd


def _assert_reference_bound(got, want, what):
    got, want = got.float().cpu(), want.float().cpu()
    excess = (got - want).abs() - (5e-2 + 1e-2 * want.abs())
    assert float(excess.max()) <= 0, (f"{what}: a logit is {float(excess.max()):.3e} beyond atol 5e-2 / rtol 1e-2 "
                                      f"(max |diff| {float((got - want).abs().max()):.3e}, max |want| {float(want.abs().max()):.2f})")


def test_released_layout_checkpoint_loads_and_generates(dev, tmp_path):
    from based_amd.mixers.linear_attention import LinearAttention
    from based_amd.mixers.slide_attention import SlidingAttention
    from based_amd.stack import GPTLMHeadModel

    cfg = released_config()
    sd = released_state_dict(cfg)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    torch.save({"model." + k: v for k, v in sd.items()}, tmp_path / "pytorch_model.bin")

    print("released-layout checkpoint: load", flush=True)
    model = GPTLMHeadModel.from_pretrained_local(str(tmp_path), device=dev, dtype=torch.bfloat16).eval()
    swa = model.transformer.layers[2].mixer
    lin = model.transformer.layers[1].mixer
    assert isinstance(swa, SlidingAttention) and swa.window == (128, 0) and swa.rotary_emb_dim == 64
    assert all(layer.supports_decode_step() for layer in model.transformer.layers)   # single-token steps take the fused path
    assert isinstance(lin, LinearAttention) and lin.eps == 1e-6     # the "fla" regulariser
    assert not hasattr(model.transformer.embeddings, "position_embeddings")
    for k, v in model.state_dict().items():
        assert torch.equal(v.cpu(), sd[k]), k                        # every tensor landed where its name says

    sd32 = {k: v.float() for k, v in sd.items()}
    B, P, n_new = 2, 300, 12      # the prompt crosses 128, 129, 256 and 257 tokens: every phase of the three-block key ring
    ids = torch.randint(1, VOCAB, (B, P), generator=torch.Generator().manual_seed(2))
    print("released-layout checkpoint: prefill", flush=True)
    with torch.inference_mode():
        logits = model(ids.to(dev)).logits
    want = O.stack_forward(ids, sd32, cfg)
    _assert_reference_bound(logits, want, "prefill logits")
    # the oracle does read the window from the config (one key more or less moves its logits); the exact edge
    # of the window is pinned at kernel level in test_swa_gpu.py::test_window_edges_are_exact
    for wrong in (254, 258):
        bad = dict(cfg, alt_mixer_2=dict(cfg["alt_mixer_2"], window_size=wrong))
        assert float((O.stack_forward(ids, sd32, bad)[:, 200:] - want[:, 200:]).abs().max()) > 1e-4

    print("released-layout checkpoint: generate", flush=True)
    out = model.generate(input_ids=ids.to(dev), max_length=P + n_new, return_dict_in_generate=True, output_scores=True,
                         top_k=1)
    seqs = out.sequences.cpu()
    for i, sc in enumerate(out.scores):
        _assert_reference_bound(sc, O.stack_forward(seqs[:, : P + i], sd32, cfg)[:, -1], f"cached decode step {i}")

    # the same request through the recorded decode graph (device-side positions feed the 129-row window
    # step and its rotary): same tokens, logits equal to bf16 noise
    print("released-layout checkpoint: graph decode", flush=True)
    graphed = model.generate(input_ids=ids.to(dev), max_length=P + n_new, return_dict_in_generate=True,
                             output_scores=True, top_k=1, cg=True)
    assert torch.equal(graphed.sequences.cpu(), seqs)
    for i, (a, b) in enumerate(zip(graphed.scores, out.scores)):
        err = float((a.float() - b.float()).norm() / b.float().norm())
        assert err < 1e-3, f"graph step {i}: rel-L2 {err:.2e} against eager"


def test_released_360m_shape_builds_with_window_256(dev):
    """The full-width released configuration: constructs, runs a 300-token prefill and two decode
    steps; cached logits equal a fresh parallel forward at the reference's bound."""
    from based_amd.stack import GPTLMHeadModel, based_360m_released_config

    torch.manual_seed(0)
    model = GPTLMHeadModel(based_360m_released_config(n_layer=8), device=dev, dtype=torch.bfloat16).eval()
    ids = torch.randint(0, 50277, (2, 300), generator=torch.Generator().manual_seed(4)).to(dev)
    out = model.generate(input_ids=ids, max_length=303, return_dict_in_generate=True, output_scores=True, top_k=1)
    with torch.inference_mode():
        for i in range(3):
            ref = model(out.sequences[:, : 300 + i]).logits[:, -1]
            _assert_reference_bound(out.scores[i], ref, f"cached step {i} vs parallel")


def test_released_1b_shape_head_dim_112(dev, tmp_path):
    """The released 1B / 1.3B shape (train/configs/experiment/reference/based-1b.yaml:72-125:
    n_embd 1792 over 16 heads = head dim 112 for BOTH attention mixers, window_size 256, rotary over
    the whole head, n_inner 2 x n_embd), narrow in depth and vocabulary: loaded from the released
    layout, prefill and every cached step against the oracle composition at the reference's bound,
    eagerly and through the recorded decode graph.  Head dim 112 must take the MFMA kernels and the
    fused single-token path (no torch-side rotary, nothing that raises under device positions)."""
    from based_amd.mixers.linear_attention import LinearAttention
    from based_amd.mixers.slide_attention import SlidingAttention
    from based_amd.stack import GPTLMHeadModel

    cfg = released_config(N_EMBD=1792, N_HEAD=16, N_LAYER=4)
    sd = released_state_dict(cfg, seed=19)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    torch.save({"model." + k: v for k, v in sd.items()}, tmp_path / "pytorch_model.bin")
    print("1B-shape checkpoint: load", flush=True)
    model = GPTLMHeadModel.from_pretrained_local(str(tmp_path), device=dev, dtype=torch.bfloat16).eval()
    swa, lin = model.transformer.layers[2].mixer, model.transformer.layers[1].mixer
    assert isinstance(swa, SlidingAttention) and swa.head_dim == 112 and swa.rotary_emb_dim == 112 and swa.window == (128, 0)
    assert isinstance(lin, LinearAttention) and lin.head_dim == 112
    assert all(layer.supports_decode_step() for layer in model.transformer.layers)

    sd32 = {k: v.float() for k, v in sd.items()}
    B, P, n_new = 2, 270, 6
    ids = torch.randint(1, VOCAB, (B, P), generator=torch.Generator().manual_seed(5))

    def check(got, seq, last_only, what):
        """At this width the logits reach +-4.5, where one bf16 step is 0.03: the element-wise bound
        of the reference's 256-wide test model is widened by what rounding alone does to the SAME
        composition evaluated with bf16 activations on the CPU, and the GPU model must sit as close
        to the fp32 statement as that composition does."""
        exact = O.stack_forward(seq, sd32, cfg)
        rounded = O.stack_forward(seq, sd32, cfg, dtype=torch.bfloat16).float()
        if last_only:
            exact, rounded = exact[:, -1], rounded[:, -1]
        got = got.float().cpu()
        noise = float((rounded - exact).abs().max())
        excess = (got - exact).abs() - (5e-2 + 1e-2 * exact.abs() + noise)
        e_gpu = float((got - exact).norm() / exact.norm())
        e_cpu = float((rounded - exact).norm() / exact.norm())
        print(f"{what}: rel-L2 to the fp32 statement GPU {e_gpu:.4f} / CPU bf16 composition {e_cpu:.4f}; "
              f"max |diff| GPU {float((got - exact).abs().max()):.4f} / CPU {noise:.4f}", flush=True)
        assert float(excess.max()) <= 0, f"{what}: a logit is {float(excess.max()):.3e} beyond the bound"
        assert e_gpu < 1.5 * e_cpu + 2e-3, f"{what}: rel-L2 {e_gpu:.4f} against {e_cpu:.4f} from rounding alone"

    print("1B-shape checkpoint: prefill", flush=True)
    with torch.inference_mode():
        logits = model(ids.to(dev)).logits
    check(logits, ids, False, "prefill logits")
    print("1B-shape checkpoint: generate", flush=True)
    out = model.generate(input_ids=ids.to(dev), max_length=P + n_new, return_dict_in_generate=True, output_scores=True,
                         top_k=1)
    seqs = out.sequences.cpu()
    for i, sc in enumerate(out.scores):
        check(sc, seqs[:, : P + i], True, f"cached decode step {i}")
    print("1B-shape checkpoint: graph decode", flush=True)
    graphed = model.generate(input_ids=ids.to(dev), max_length=P + n_new, return_dict_in_generate=True,
                             output_scores=True, top_k=1, cg=True)
    assert torch.equal(graphed.sequences.cpu(), seqs)
    for i, (a, b) in enumerate(zip(graphed.scores, out.scores)):
        err = float((a.float() - b.float()).norm() / b.float().norm())
        assert err < 1e-3, f"graph step {i}: rel-L2 {err:.2e} against eager"
