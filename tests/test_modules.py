"""CPU tests of the host-side mirror of the reference's module layer: CatsMLP switches, histogram calibration and
its on-disk format, and the decoder used for the end-to-end decode measurement."""
import math

import pytest
import torch
import torch.nn.functional as F

from cats_amd import decoder as dec
from cats_amd import mlp as cm


def tiny_model(layers=4, hidden=64, inter=64, heads=4, vocab=97, max_len=48, dtype=torch.float32):
    cfg = dec.DecoderConfig(hidden_size=hidden, intermediate_size=inter, num_layers=layers, num_heads=heads, vocab_size=vocab, max_len=max_len)
    return dec.LlamaDecoder(cfg, dtype, "cpu", seed=0, init_std=0.2).eval()


def test_cats_mlp_dense_masked_branch_matches_oracle(oracle):
    torch.manual_seed(0)
    m = cm.CatsMLP(64, 96, dtype=torch.float32)
    x = torch.randn(2, 1, 64)
    m.is_profile, m.sp_method, m.dead_threshold = True, 0, 0.08
    y, _, _ = oracle.torch_cats_mlp(x, m.gate_proj.weight, m.up_proj.weight, m.down_proj.weight, 0.08)
    torch.testing.assert_close(m(x), y)
    # prefill shape goes the same way; the non-profile path with the kill switch is the same function
    xp = torch.randn(1, 5, 64)
    m2 = cm.CatsMLP(64, 96, dtype=torch.float32)
    m2.load_state_dict(m.state_dict())
    m2.kill_sparse_swish_outputs, m2.dead_threshold = True, 0.08
    torch.testing.assert_close(m(xp), m2(xp))
    # threshold 0 with the kill switch off is the plain SwiGLU MLP
    m2.kill_sparse_swish_outputs = False
    torch.testing.assert_close(m2(xp), oracle.torch_dense_mlp(xp, m.gate_proj.weight, m.up_proj.weight, m.down_proj.weight))
    # sp_mask branch uses SparseSiLU on the masked gate
    mask = (torch.rand(96) > 0.5).float()
    m.sparse_act_fn.set_new_threshold(0.08)   # the reference updates it only through set_sparse_threshold
    want = F.linear(oracle.torch_sparse_silu(F.linear(xp, m.gate_proj.weight) * mask, 0.08) * F.linear(xp, m.up_proj.weight), m.down_proj.weight)
    torch.testing.assert_close(m(xp, sp_mask=mask), want)


def test_kernel_methods_fail_loudly_without_gpu():
    m = cm.CatsMLP(64, 96, dtype=torch.float16).prepare_decode(3)
    with pytest.raises(RuntimeError):
        m(torch.zeros(1, 1, 64, dtype=torch.float16))
    m.wdown_t = None
    with pytest.raises(RuntimeError, match="wdown_t"):
        m(torch.zeros(1, 1, 64, dtype=torch.float16))


def test_histogram_calibration_roundtrip(tmp_path, oracle):
    model = tiny_model()
    cm.activate_stats(model)
    g = torch.Generator().manual_seed(0)
    toks = torch.randint(0, 97, (3, 16), generator=g)
    model.reset_cache(3)
    model(toks, torch.arange(16))
    for layer in model.layers:
        assert float(layer.mlp.post_act_hist_counts.sum()) == 3 * 16 * 64
        assert float(layer.mlp.pre_act_hist_counts.sum()) == 3 * 16 * 64
    want = [float(oracle.torch_get_threshold(l.mlp.histogram_bins, l.mlp.post_act_hist_counts, 0.5)) for l in model.layers]
    path = str(tmp_path / "hist" / "act_hist.pt")
    cm.save_act_hist(model, path)
    cm.set_sparse_threshold(model, 0.5)
    assert cm.get_thresholds(model) == want
    # the file is {layer: (bins, pre, post)} of plain tensors and loads without unpickling code
    blob = torch.load(path, weights_only=True)
    assert sorted(blob) == [0, 1, 2, 3] and all(len(v) == 3 and v[0].numel() == 1000 and v[2].numel() == 999 for v in blob.values())
    other = tiny_model()
    cm.activate_stats(other)
    cm.load_act_hist(other, path)
    cm.set_sparse_threshold(other, 0.5)
    assert cm.get_thresholds(other) == want
    # achieved sparsity on the calibration data is within a bin of the target
    cm.set_thresholds(other, want)
    assert all(l.mlp.kill_sparse_swish_outputs for l in other.layers)


def test_apply_cats_mlp_shares_projections():
    model = tiny_model()
    old = [l.mlp.gate_proj for l in model.layers]
    for l in model.layers:      # stand-in for an HF MLP: any module with the three projections
        plain = torch.nn.Module()
        plain.gate_proj, plain.up_proj, plain.down_proj = l.mlp.gate_proj, l.mlp.up_proj, l.mlp.down_proj
        l.mlp = plain
    cm.apply_cats_mlp(model, dead_threshold=0.1)
    assert all(isinstance(l.mlp, cm.CatsMLP) and l.mlp.gate_proj is o for l, o in zip(model.layers, old))
    cm.prepare_decode(model, 2)
    assert all(l.mlp.is_profile and l.mlp.sp_method == 2 and l.mlp.wdown_t.shape == (64, 64) for l in model.layers)
    assert torch.equal(model.layers[0].mlp.wdown_t, model.layers[0].mlp.down_proj.weight.t())


def test_decoder_incremental_equals_full_sequence():
    model = tiny_model()
    g = torch.Generator().manual_seed(1)
    toks = torch.randint(0, 97, (1, 12), generator=g)
    model.reset_cache(1)
    full = model(toks, torch.arange(12))
    model.reset_cache(1)
    model(toks[:, :5], torch.arange(5))
    for i in range(5, 12):
        step = model(toks[:, i:i + 1], torch.tensor([i]))
        torch.testing.assert_close(step[:, 0], full[:, i], rtol=1e-4, atol=1e-5)


def test_decoder_matches_hf_llama_on_the_reference_debug_shape():
    """Second opinion on RoPE / attention / norm conventions: the installed transformers Llama (third party, not the
    reference) built from an in-code config -- hidden 64, intermediate 64, 4 layers, the reference's own debug shape
    (experiments/pretrain_sparse_model.py:92-96)."""
    tr = pytest.importorskip("transformers")
    try:
        hf_cfg = tr.LlamaConfig(hidden_size=64, intermediate_size=64, num_hidden_layers=4, num_attention_heads=4, num_key_value_heads=4,
                                vocab_size=97, max_position_embeddings=48, rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=False,
                                attention_bias=False, mlp_bias=False, attn_implementation="eager")
        hf = tr.LlamaForCausalLM(hf_cfg).eval()
    except Exception as e:  # pragma: no cover - depends on the installed transformers
        pytest.skip(f"transformers Llama not constructible here: {e}")
    model = tiny_model()
    sd = {"model.embed_tokens.weight": model.embed_tokens.weight, "model.norm.weight": model.norm.weight, "lm_head.weight": model.lm_head.weight}
    for i, l in enumerate(model.layers):
        p = f"model.layers.{i}."
        sd.update({p + "input_layernorm.weight": l.input_layernorm.weight, p + "post_attention_layernorm.weight": l.post_attention_layernorm.weight,
                   p + "self_attn.q_proj.weight": l.self_attn.q_proj.weight, p + "self_attn.k_proj.weight": l.self_attn.k_proj.weight,
                   p + "self_attn.v_proj.weight": l.self_attn.v_proj.weight, p + "self_attn.o_proj.weight": l.self_attn.o_proj.weight,
                   p + "mlp.gate_proj.weight": l.mlp.gate_proj.weight, p + "mlp.up_proj.weight": l.mlp.up_proj.weight,
                   p + "mlp.down_proj.weight": l.mlp.down_proj.weight})
    missing = hf.load_state_dict(sd, strict=False)
    assert not [k for k in missing.missing_keys if "rotary" not in k]
    g = torch.Generator().manual_seed(2)
    toks = torch.randint(0, 97, (2, 10), generator=g)
    with torch.no_grad():
        want = hf(input_ids=toks).logits
    model.reset_cache(2)
    got = model(toks, torch.arange(10))
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-4)


def test_greedy_decode_dense_vs_masked_threshold_zero():
    """With a negative threshold the dense-masked CATS path must reproduce the dense model's greedy tokens."""
    model = tiny_model()
    g = torch.Generator().manual_seed(3)
    prompt = torch.randint(0, 97, (1, 6), generator=g)
    model.set_mlp_mode("dense")
    dense_tokens, _ = _greedy_cpu(model, prompt, 8)
    for l in model.layers:
        l.mlp.dead_threshold = -1.0
    model.set_mlp_mode("cats_torch")
    cats_tokens, _ = _greedy_cpu(model, prompt, 8)
    assert torch.equal(dense_tokens, cats_tokens)


def _greedy_cpu(model, prompt, n):
    model.reset_cache(1)
    P = prompt.shape[1]
    logits = model(prompt, torch.arange(P))
    tok = logits[:, -1].argmax(-1, keepdim=True)
    out = [int(tok)]
    for i in range(n - 1):
        logits = model(tok, torch.tensor([P + i]))
        tok = logits[:, -1].argmax(-1, keepdim=True)
        out.append(int(tok))
    return torch.tensor(out), logits
