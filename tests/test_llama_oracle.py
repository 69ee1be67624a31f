"""Pins oracle/llama_oracle.py (the decode step around the compressed linears) against the
third-party model code the reference patches its modules into: `transformers`' Llama
(bitstack/utils/model_utils.py:189-205 builds it with AutoModelForCausalLM.from_config).
A tiny random model, fp32 there, float64 here; token-by-token decode here against one causal
pass there, so a wrong rotation pairing, cache index, head grouping, norm or residual shows up."""
import numpy as np
import pytest
import torch

from oracle import llama_oracle as lo

transformers = pytest.importorskip("transformers")
THETA = 500000.0


@pytest.fixture(scope="module")
def tiny():
    from transformers import LlamaConfig, LlamaForCausalLM
    cfg = LlamaConfig(hidden_size=256, intermediate_size=384, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, head_dim=64, vocab_size=50, rope_theta=THETA, rms_norm_eps=1e-5,
                      max_position_embeddings=32, tie_word_embeddings=False, attention_bias=False, mlp_bias=False)
    torch.manual_seed(3)
    model = LlamaForCausalLM(cfg).float().eval()
    with torch.no_grad():
        for name, p in model.named_parameters():          # norms away from 1 so a dropped weight is visible
            if "norm" in name:
                p.copy_(1.0 + 0.3 * torch.randn_like(p))
    return cfg, model


def test_decode_steps_match_transformers_causal_pass(tiny):
    cfg, model = tiny
    ids = torch.tensor([[7, 3, 41, 3, 19, 0, 28, 11, 5]])
    with torch.no_grad():
        ref = model(ids).logits[0].double().numpy()
    weights = {k: v.detach().double().numpy() for k, v in model.state_dict().items()}
    orc = lo.LlamaOracle(weights, cfg.num_hidden_layers, cfg.num_attention_heads, cfg.num_key_value_heads,
                         cfg.head_dim, THETA, cfg.rms_norm_eps, max_len=16)
    for p, tok in enumerate(ids[0].tolist()):
        got = orc.step(tok)
        assert np.abs(got - ref[p]).max() <= 2e-4 * max(1.0, np.abs(ref[p]).max()), p


def test_pieces_against_transformers_functions(tiny):
    from transformers.models.llama.modeling_llama import LlamaRMSNorm, apply_rotary_pos_emb, LlamaRotaryEmbedding
    cfg, _ = tiny
    g = torch.Generator().manual_seed(0)
    x = torch.randn(3, 256, generator=g, dtype=torch.float64)
    norm = LlamaRMSNorm(256, eps=1e-5).double()
    with torch.no_grad():
        norm.weight.copy_(torch.randn(256, generator=g, dtype=torch.float64))
        want = norm(x).numpy()
    assert np.allclose(lo.rmsnorm(x.numpy(), norm.weight.detach().numpy(), 1e-5), want, rtol=1e-5, atol=1e-6)

    rot = LlamaRotaryEmbedding(config=cfg)
    pos = torch.tensor([[0, 1, 5, 9]])
    cos, sin = rot(torch.zeros(1, 4, 256), pos)              # [1, 4, d] (halves repeated)
    q = torch.randn(1, 4, 4, 64, generator=g)                # [b, heads, seq, d]
    k = torch.randn(1, 2, 4, 64, generator=g)
    q2, k2 = apply_rotary_pos_emb(q, k, cos, sin)
    c, s = lo.rope_tables(16, 64, THETA)
    for j, p in enumerate(pos[0].tolist()):
        assert np.allclose(lo.rope(q[0, :, j].numpy(), c[p], s[p]), q2[0, :, j].numpy(), atol=2e-6)
        assert np.allclose(lo.rope(k[0, :, j].numpy(), c[p], s[p]), k2[0, :, j].numpy(), atol=2e-6)


def test_attention_closed_forms():
    # one cached position: softmax over one score is 1, the output is v itself
    q = np.random.default_rng(0).normal(size=(4, 8))
    kc = np.random.default_rng(1).normal(size=(2, 5, 8))
    vc = np.random.default_rng(2).normal(size=(2, 5, 8))
    out = lo.attention_decode(q, kc, vc, 1)
    assert np.allclose(out[0], vc[0, 0]) and np.allclose(out[3], vc[1, 0])
    # identical keys: uniform weights, the output is the mean of v
    kc[:] = kc[:, :1]
    out = lo.attention_decode(q, kc, vc, 5)
    assert np.allclose(out[1], vc[0].mean(0)) and np.allclose(out[2], vc[1].mean(0))
    assert np.isclose(lo.silu(0.0), 0.0) and np.isclose(lo.silu(50.0), 50.0) and np.isclose(lo.silu(1.0), 1 / (1 + np.exp(-1.0)))


def test_rope_frequencies_with_llama3_scaling_match_transformers():
    """The decoder's RoPE tables for the released Llama-3.1 / 3.2 configurations (rope_type "llama3")
    against the library the reference runs those models through; plain and linear scaling too, and
    an unknown type is refused instead of silently giving default tables."""
    import pytest
    from transformers import LlamaConfig
    from transformers.modeling_rope_utils import ROPE_INIT_FUNCTIONS
    from bitstack_amd.utils.llama_decode import rope_inv_freq
    for d, theta, sc in [(128, 500000.0, dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                               original_max_position_embeddings=8192)),
                         (64, 500000.0, dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                              original_max_position_embeddings=8192)),
                         (64, 10000.0, dict(rope_type="linear", factor=4.0))]:
        cfg = LlamaConfig(hidden_size=d * 2, num_attention_heads=2, num_hidden_layers=1, intermediate_size=64, vocab_size=8,
                          head_dim=d, max_position_embeddings=131072, rope_parameters=dict(sc, rope_theta=theta))
        want, att = ROPE_INIT_FUNCTIONS[sc["rope_type"]](cfg, "cpu")
        got = rope_inv_freq(d, theta, sc)
        assert att == 1.0 and got.dtype == torch.float32
        assert torch.allclose(got, want.float(), rtol=1e-6, atol=0), sc
        plain = rope_inv_freq(d, theta, None)
        assert torch.equal(plain[0:1], got[0:1]) or sc["rope_type"] == "linear"     # the fastest frequency is untouched by llama3
        assert not torch.equal(plain, got)
    assert torch.allclose(rope_inv_freq(8, 100.0), torch.tensor([1.0, 100 ** -0.25, 100 ** -0.5, 100 ** -0.75]))
    assert torch.equal(rope_inv_freq(8, 100.0, {"rope_type": "default"}), rope_inv_freq(8, 100.0))
    with pytest.raises(ValueError, match="yarn"):
        rope_inv_freq(64, 10000.0, {"rope_type": "yarn", "factor": 2.0})
