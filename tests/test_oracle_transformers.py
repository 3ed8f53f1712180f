"""Pins of the oracle's rotary, RMSNorm and decoder functions against the library the reference itself calls
for them: transformers' LlamaRotaryEmbedding / apply_rotary_pos_emb (fused_attention.py:7,101-102 of the
reference), LlamaRMSNorm and LlamaForCausalLM (the model src/gptq_triton/__init__.py:32-52 builds and patches).
The installed transformers is read through its public classes, in float32 on the CPU.  Two pins of the decoder
reference that need no library follow at the end."""
import math

import numpy as np
import pytest
import torch

from oracle import decoder_ref
from oracle import gptq_oracle as O

transformers = pytest.importorskip("transformers")


def hf_config(**kw):
    from transformers import LlamaConfig
    base = dict(hidden_size=256, intermediate_size=768, num_hidden_layers=2, num_attention_heads=2,
                num_key_value_heads=2, vocab_size=320, max_position_embeddings=512, rms_norm_eps=1e-6,
                rope_theta=10000.0, hidden_act="silu", attention_bias=False, mlp_bias=False, tie_word_embeddings=False)
    base.update(kw)
    cfg = LlamaConfig(**base)
    cfg._attn_implementation = "eager"
    return cfg


def test_rotary_tables_equal_transformers_rotary_embedding():
    from transformers.models.llama.modeling_llama import LlamaRotaryEmbedding
    cfg = hf_config(hidden_size=4096, num_attention_heads=32, num_key_value_heads=32, max_position_embeddings=2048)
    rope = LlamaRotaryEmbedding(cfg)
    pos = torch.arange(2048)[None, :]
    cos_hf, sin_hf = rope(torch.zeros(1, 2048, 128, dtype=torch.float32), pos)   # [1, S, 128]: halves repeated
    cos, sin = O.rotary_tables(2048, 128, 10000.0)
    cos_hf, sin_hf = cos_hf[0].double().numpy(), sin_hf[0].double().numpy()
    # column j >= 64 of the library's table repeats column j - 64
    assert np.array_equal(cos_hf[:, :64], cos_hf[:, 64:]) and np.array_equal(sin_hf[:, :64], sin_hf[:, 64:])
    # the frequencies: the library's float32 pow leaves inv_freq within one ulp of float32(base^(-2i/D)), the
    # correctly rounded value the oracle (and the table kernel) use
    expo = np.arange(0, 128, 2, dtype=np.float64) / 128.0
    inv = (1.0 / np.power(10000.0, expo)).astype(np.float32)
    inv_hf = rope.inv_freq.numpy()
    assert (np.abs(inv_hf.astype(np.float64) - inv) <= np.spacing(inv)).all()
    # with the library's own frequencies the oracle's formula - float32 angle = float32(p) * inv_freq, cos/sin of
    # it rounded once - reproduces the library's float32 tables to float32 rounding
    cos_l, sin_l = O.rotary_tables(2048, 128, 10000.0, inv_freq=inv_hf)
    assert np.abs(cos_hf[:, :64] - cos_l).max() <= 2.5e-7 and np.abs(sin_hf[:, :64] - sin_l).max() <= 2.5e-7
    # and the oracle's own tables differ from the library's by no more than that one ulp of frequency times the
    # position, plus the rounding of the float32 angle that it can flip (together 2.5e-4 at position 2047) - the
    # spread the library itself shows between pow implementations
    theta = (np.arange(2048, dtype=np.float32)[:, None] * inv[None, :]).astype(np.float32)
    bound = np.arange(2048)[:, None] * np.spacing(inv)[None, :] + np.spacing(theta) + 2.5e-7
    assert (np.abs(cos_hf[:, :64] - cos) <= bound).all() and (np.abs(sin_hf[:, :64] - sin) <= bound).all()


def test_apply_rotary_equals_transformers_apply_rotary_pos_emb():
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb
    rng = np.random.default_rng(0)
    b, h, s, d = 2, 3, 17, 128
    q = rng.standard_normal((b, h, s, d)).astype(np.float32)
    k = rng.standard_normal((b, h, s, d)).astype(np.float32)
    pos = rng.integers(0, 2048, size=(b, s))
    cos, sin = O.rotary_tables(2048, d)
    c, sn = cos[pos], sin[pos]                                   # [B, S, 64]
    cf = torch.from_numpy(np.concatenate([c, c], -1))            # the library's layout: halves repeated
    sf = torch.from_numpy(np.concatenate([sn, sn], -1))
    q_hf, k_hf = apply_rotary_pos_emb(torch.from_numpy(q), torch.from_numpy(k), cf, sf, unsqueeze_dim=1)
    q_or = O.apply_rotary(q, c[:, None], sn[:, None])
    k_or = O.apply_rotary(k, c[:, None], sn[:, None])
    # same formula (sign convention, pairing d / d + 64); float32 products against float64
    assert np.abs(q_hf.numpy() - q_or).max() <= 1e-6 and np.abs(k_hf.numpy() - k_or).max() <= 1e-6
    # a swapped sign or a (2i, 2i+1) pairing is far outside that
    wrong = np.concatenate([q[..., :64] * c[:, None] + q[..., 64:] * sn[:, None], q[..., 64:] * c[:, None] - q[..., :64] * sn[:, None]], -1)
    assert np.abs(q_hf.numpy() - wrong).max() > 0.1


@pytest.mark.parametrize("eps", [1e-6, 1e-5])
def test_rmsnorm_ref_equals_transformers_rmsnorm(eps):
    from transformers.models.llama.modeling_llama import LlamaRMSNorm
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((5, 512)) * 3).astype(np.float16)
    w = (1 + 0.1 * rng.standard_normal(512)).astype(np.float16)
    norm = LlamaRMSNorm(512, eps=eps).half()
    norm.weight.data = torch.from_numpy(w)
    got = norm(torch.from_numpy(x)).detach().numpy()       # statistics in float32, cast to fp16, fp16 multiply by the weight
    ref = O.rmsnorm_ref(x, w, eps)
    # the same rounding order: equal except where the float32 normalised value sits within float32 error of an fp16 tie
    diff = np.abs(got.astype(np.float32) - ref.astype(np.float32))
    assert (diff <= np.spacing(np.abs(ref).astype(np.float16)).astype(np.float32)).all()
    assert (got.view(np.uint16) == ref.view(np.uint16)).mean() > 0.999


def lite_config(**kw):
    """The same tiny model as the plain record the oracle's decoder reads its fields from."""
    from gptq_triton_amd.fused_attention import LlamaConfigLite
    cfg = LlamaConfigLite(hidden_size=256, num_attention_heads=2, max_position_embeddings=512, intermediate_size=768,
                          num_hidden_layers=2, vocab_size=320, rms_norm_eps=1e-6, rope_theta=10000.0)
    for k, v in kw.items():
        setattr(cfg, k, v)
    return cfg


def _tiny_state(cfg, groupsize, seed):
    """An UNFUSED checkpoint state_dict of random packed weights for a tiny model."""
    rng = np.random.default_rng(seed)
    h, inter = cfg.hidden_size, cfg.intermediate_size
    state = {"model.embed_tokens.weight": torch.from_numpy(rng.standard_normal((cfg.vocab_size, h)).astype(np.float32)).half(),
             "lm_head.weight": torch.from_numpy((rng.standard_normal((cfg.vocab_size, h)) * 0.05).astype(np.float32)).half(),
             "model.norm.weight": torch.from_numpy((1 + 0.1 * rng.standard_normal(h)).astype(np.float32)).half()}
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        for name in ("input_layernorm", "post_attention_layernorm"):
            state[p + name + ".weight"] = torch.from_numpy((1 + 0.1 * rng.standard_normal(h)).astype(np.float32)).half()
        for name, (k, n) in (("self_attn.q_proj", (h, h)), ("self_attn.k_proj", (h, h)), ("self_attn.v_proj", (h, h)),
                             ("self_attn.o_proj", (h, h)), ("mlp.gate_proj", (h, inter)), ("mlp.up_proj", (h, inter)),
                             ("mlp.down_proj", (inter, h))):
            L = O.make_layer(k, n, groupsize, seed=int(rng.integers(1 << 30)))
            # scales sized so that activations stay O(1) through the layers
            L["scales"] = (L["scales"].astype(np.float32) * (4.0 / math.sqrt(k))).astype(np.float16)
            for t in ("qweight", "qzeros", "scales"):
                state[p + name + "." + t] = torch.from_numpy(L[t])
    return state


@pytest.mark.parametrize("groupsize", [-1, 128])
def test_decoder_ref_equals_transformers_llama(groupsize):
    from transformers import LlamaForCausalLM
    cfg = lite_config()
    state = _tiny_state(cfg, groupsize, seed=3)
    torch.manual_seed(0)
    model = LlamaForCausalLM(hf_config()).float().eval()
    sd = {}
    for k, v in state.items():
        if k.endswith(".qweight"):
            prefix = k[:-len(".qweight")]
            sd[prefix + ".weight"] = decoder_ref.dequant(state, prefix, groupsize).t().contiguous()   # nn.Linear holds [out, in]
        elif not k.endswith((".qzeros", ".scales")):
            sd[k] = v.float()
    missing, unexpected = model.load_state_dict(sd, strict=False)
    assert not unexpected and all("rotary" in m or "inv_freq" in m for m in missing), (missing, unexpected)
    ids = torch.randint(0, cfg.vocab_size, (2, 23))
    with torch.no_grad():
        want = model(ids).logits
    got = decoder_ref.forward(state, cfg, groupsize, ids)
    scale = want.abs().max().item()
    assert scale > 0.5, "logits too small to say anything"
    assert (got - want).abs().max().item() <= 1e-4 * max(scale, 1.0)


def test_decoder_ref_is_causal():
    """Logits at position t do not change when tokens after t change."""
    cfg = lite_config()
    state = _tiny_state(cfg, 128, seed=5)
    torch.manual_seed(1)
    a = torch.randint(0, cfg.vocab_size, (1, 20))
    b = a.clone()
    b[:, 12:] = torch.randint(0, cfg.vocab_size, (1, 8))
    la, lb = decoder_ref.forward(state, cfg, 128, a), decoder_ref.forward(state, cfg, 128, b)
    assert torch.equal(la[:, :12], lb[:, :12])
    assert not torch.equal(la[:, 12:], lb[:, 12:])


def test_decoder_ref_with_silent_blocks_is_head_of_norm_of_embedding():
    """With o_proj and down_proj decoding to zero the residual stream stays the embedding: logits = lm_head(norm(embed))."""
    cfg = lite_config(num_hidden_layers=1)
    state = _tiny_state(cfg, -1, seed=7)
    for name in ("self_attn.o_proj", "mlp.down_proj"):
        p = f"model.layers.0.{name}."
        # q = z + 1 everywhere: every weight decodes to (q - (z + 1)) * s = 0
        z = O.unpack_qzeros(state[p + "qzeros"].numpy())                     # [G = 1, N] stored zeros
        z = np.where(z + 1 <= 15, z, 0)                                      # stored zero 15 would need q = 16
        q = np.repeat(z + 1, state[p + "qweight"].shape[0] * 8, axis=0)
        state[p + "qzeros"] = torch.from_numpy(O.pack_qzeros(z))
        state[p + "qweight"] = torch.from_numpy(O.pack_qweight(q))
        assert not decoder_ref.dequant(state, p[:-1], -1).any()
    ids = torch.randint(0, cfg.vocab_size, (2, 9))
    got = decoder_ref.forward(state, cfg, -1, ids)
    e = state["model.embed_tokens.weight"].float()[ids]
    want = decoder_ref.rmsnorm(e, state["model.norm.weight"], cfg.rms_norm_eps) @ state["lm_head.weight"].float().t()
    assert torch.allclose(got, want, rtol=0, atol=1e-5)
