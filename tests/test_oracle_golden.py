"""Pins the oracle's composed layer (fused-qkv head layout, rotary, causal attention, pre-norm
residuals, final norm) against the golden activations held by the reference's test-suite."""

import os

import torch
import torch.nn.functional as F

import oracle

TOL = 3.0e-3  # the reference's own gate for this fixture


def _load(golden_dir):
    d = os.path.join(golden_dir, "backward_compatibility")
    gt = torch.load(os.path.join(d, "ground_truth.pt"), weights_only=True)
    sd = torch.load(os.path.join(d, "state_dict.pt"), weights_only=True)
    layer, final = {}, {}
    for k, v in sd.items():
        if k.endswith(".inv_freq"):
            continue
        if k.startswith("transformer.layer0."):
            k2 = k[len("transformer.layer0."):].replace("attention.", "self_attention.", 1) \
                if k.startswith("transformer.layer0.attention.") else k[len("transformer.layer0."):]
            k2 = k2.replace("dense_h_to_4h", "dense_in").replace("dense_4h_to_h", "dense_out")
            layer[k2] = v
        elif k.startswith("transformer.norm."):
            final[k.replace("transformer.", "")] = v
    emb = sd["transformer.embeddings.word_embeddings.weight"]
    return gt, layer, final, emb


def test_layer_golden(golden_dir):
    gt, w, final, emb = _load(golden_dir)
    spec = oracle.LayerSpec(hidden_size=16, num_attention_heads=2, sequence_length=4)
    ids = gt["input"]
    assert ids.tolist() == [[0, 1, 2, 3]]
    cu = oracle.get_cumulative_seq_lengths(ids, reset_attention_mask=False)
    pos = oracle.get_position_ids(ids, reset_position_ids=False)
    h0 = F.embedding(ids, emb)

    def err(a, key):
        return float((a.detach() - gt[key].detach()).abs().max())

    assert err(h0, "hidden_states_embedding") < TOL
    assert err(oracle.layer_norm(h0, w["input_layernorm.weight"], w["input_layernorm.bias"]),
               "hidden_states_input_layernorm") < TOL
    att = oracle.attention_block(spec, w, h0, cu, pos)
    assert err(att, "hidden_states_attention") < 1e-4
    assert err(oracle.layer_norm(att, w["post_attention_layernorm.weight"], w["post_attention_layernorm.bias"]),
               "hidden_states_post_attention_layernorm") < TOL
    assert err(oracle.mlp_block(spec, w, att), "hidden_states_mlp") < 1e-4
    out = oracle.transformer_layer(spec, w, h0, cu, pos)
    assert err(out, "hidden_states_layer0") < TOL
    fn = oracle.final_norm(spec, final, out)
    assert err(fn, "hidden_states_norm") < TOL
    assert err(F.linear(fn, emb), "output_logits") < TOL


def test_golden_detects_plausible_mistakes(golden_dir):
    """The fixture separates the right head layout / rotary pairing / mask from near misses."""
    gt, w, final, emb = _load(golden_dir)
    h0 = F.embedding(gt["input"], emb)
    cu = torch.tensor([0, 4], dtype=torch.int32)
    pos = torch.arange(4).unsqueeze(0)
    good = oracle.LayerSpec(hidden_size=16, num_attention_heads=2, sequence_length=4)
    ref = gt["hidden_states_attention"]
    for bad in (oracle.LayerSpec(hidden_size=16, num_attention_heads=2, sequence_length=4, causal=False),
                oracle.LayerSpec(hidden_size=16, num_attention_heads=2, sequence_length=4, rotary="none"),
                oracle.LayerSpec(hidden_size=16, num_attention_heads=2, sequence_length=4, rotary="rotary_complex"),
                oracle.LayerSpec(hidden_size=16, num_attention_heads=2, sequence_length=4, rotary_base=500000)):
        with torch.no_grad():
            assert float((oracle.attention_block(bad, w, h0, cu, pos) - ref).abs().max()) > 4e-3
    with torch.no_grad():
        assert float((oracle.attention_block(good, w, h0, cu, pos) - ref).abs().max()) < 1e-4
