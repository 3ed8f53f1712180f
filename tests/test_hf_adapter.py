"""load_quant(use_transformers=True): the skeleton is a `transformers.LlamaForCausalLM`, as in the reference
(src/gptq_triton/__init__.py:32-52), with its linears, attention blocks and MLPs replaced by this package's modules.
The decoder layer of the installed transformers calls its attention block with a Cache object and precomputed
position embeddings; QuantLlamaAttention answers that call (and still the reference's 2023 signature)."""
import pytest
import torch

import gptq_triton_amd as G
from test_loader import make_checkpoint

transformers = pytest.importorskip("transformers")
pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("groupsize,act_order", [(-1, False), (128, False), (128, True)])
def test_quantised_checkpoint_in_a_transformers_model(tmp_path, groupsize, act_order):
    from oracle import decoder_ref
    from safetensors.torch import load_file
    cfg = make_checkpoint(tmp_path, groupsize, act_order=act_order, seed=11)
    state = load_file(str(tmp_path / "model.safetensors"))
    hf = G.load_quant(str(tmp_path), device="cuda", fuse_mlp=True, use_transformers=True)
    assert isinstance(hf, transformers.LlamaForCausalLM)
    layer = hf.model.layers[0]
    assert isinstance(layer.self_attn, G.QuantLlamaAttention) and layer.self_attn.layer_idx == 0
    assert isinstance(layer.mlp, G.QuantLlamaMLP)
    assert isinstance(hf.lm_head, torch.nn.Linear)

    torch.manual_seed(2)
    ids = torch.randint(0, cfg.vocab_size, (2, 40))
    with torch.no_grad():
        got = hf(input_ids=ids.cuda()).logits.float().cpu()
    ref = decoder_ref.forward(state, cfg, groupsize, ids)
    # the bound of test_loader.py: fp16 activations through two layers against the float32 reference decoder
    bound = 0.006
    err = (got - ref).abs()
    assert err.max().item() < bound and err.mean().item() < 1e-3, (err.max().item(), err.mean().item())

    # the same logits as this package's own decoder on the same checkpoint (same kernels; the norms differ in rounding)
    native = G.load_quant(str(tmp_path), device="cuda", fuse_mlp=True)
    mine, _ = native(ids.cuda())
    assert (mine.float().cpu() - got).abs().max().item() < bound

    # generate(): prefill, then single tokens through a transformers Cache; greedy tokens follow the argmax of the full
    # forward wherever the reference's best logit leads clearly
    prompt = ids[:, :8].cuda()
    with torch.no_grad():
        out = hf.generate(prompt, max_new_tokens=6, do_sample=False, pad_token_id=0)
    assert out.shape == (2, 14) and torch.equal(out[:, :8], prompt)
    with torch.no_grad():
        full = hf(input_ids=out[:, :-1]).logits.float()
    top2 = full.topk(2, dim=-1).values
    clear = ((top2[..., 0] - top2[..., 1]) > 2 * bound)[:, 7:]
    assert clear.float().mean() > 0.5
    assert torch.equal(full.argmax(-1)[:, 7:][clear], out[:, 8:][clear])

    # an incremental pass by hand, with a DynamicCache, equals the full forward
    cache = transformers.DynamicCache()
    with torch.no_grad():
        part = hf(input_ids=ids[:, :30].cuda(), past_key_values=cache, use_cache=True).logits
        steps = [part]
        for t in range(30, 40):
            steps.append(hf(input_ids=ids[:, t:t + 1].cuda(), past_key_values=cache, use_cache=True).logits)
    inc = torch.cat(steps, dim=1).float().cpu()
    assert (inc - got).abs().max() < 0.03 * got.abs().max()


def test_padded_batch_uses_the_mask_transformers_hands_over(tmp_path):
    """Left-padded prompts: the attention mask reaches the block as transformers built it."""
    cfg = make_checkpoint(tmp_path, 128, seed=12)
    hf = G.load_quant(str(tmp_path), device="cuda", fuse_mlp=True, use_transformers=True)
    torch.manual_seed(3)
    ids = torch.randint(1, cfg.vocab_size, (1, 12)).cuda()
    with torch.no_grad():
        alone = hf(input_ids=ids).logits[:, -1].float()
        padded = torch.cat([torch.zeros(1, 5, dtype=ids.dtype, device="cuda"), ids], dim=1)
        mask = torch.cat([torch.zeros(1, 5, dtype=torch.long, device="cuda"), torch.ones(1, 12, dtype=torch.long, device="cuda")], dim=1)
        both = hf(input_ids=padded, attention_mask=mask).logits[:, -1].float()
    assert (alone - both).abs().max() < 0.02 * alone.abs().max()


def test_reference_signature_still_answers(tmp_path):
    """The 2023 call: a (key, value) pair in, a triple out."""
    make_checkpoint(tmp_path, 128, seed=13)
    native = G.load_quant(str(tmp_path), device="cuda", fuse_mlp=True)
    attn = native.model.layers[0].self_attn
    x = torch.randn(2, 5, 256, device="cuda").half()
    out, weights, present = attn(x, use_cache=True)
    assert out.shape == (2, 5, 256) and weights is None and present[0].shape == (2, 2, 5, 128)
    out2, _, present2 = attn(x[:, :1].contiguous(), past_key_value=present, use_cache=True)
    assert out2.shape == (2, 1, 256) and present2[0].shape == (2, 2, 6, 128)


def test_preallocated_cache_without_a_mask_attends_to_written_slots_only(tmp_path):
    """A StaticCache hands back tensors of its whole capacity.  Called without a mask, the block attends to the slots
    written so far - a prompt, a chunk behind it, single tokens - exactly as with a DynamicCache."""
    make_checkpoint(tmp_path, 128, seed=14)
    hf = G.load_quant(str(tmp_path), device="cuda", fuse_mlp=True, use_transformers=True)
    attn = hf.model.layers[0].self_attn
    torch.manual_seed(4)
    x = (0.5 * torch.randn(2, 12, 256, device="cuda")).half()
    chunks = ((0, 6), (6, 10), (10, 11), (11, 12))

    def run(cache):
        outs = []
        with torch.no_grad():
            for a, b in chunks:
                pos = torch.arange(a, b, device="cuda").unsqueeze(0)
                out, _ = attn(x[:, a:b].contiguous(), position_ids=pos, past_key_values=cache,
                              position_embeddings=(None, None), cache_position=pos[0])
                outs.append(out)
        return torch.cat(outs, dim=1)

    dyn = run(transformers.DynamicCache())
    static = run(transformers.StaticCache(config=hf.config, max_cache_len=32))
    assert torch.equal(dyn, static)
    with torch.no_grad():
        whole, _ = attn(x, position_ids=torch.arange(12, device="cuda").unsqueeze(0), past_key_values=None,
                        position_embeddings=(None, None))
    assert (whole.float() - dyn.float()).abs().max() < 2e-3 + 1e-2 * whole.float().abs().max()


def test_generate_with_a_static_cache(tmp_path):
    """transformers builds the mask for a preallocated cache itself; greedy tokens equal those of the default cache.
    (disable_compile: with a preallocated cache generate() would otherwise hand the forward pass to torch.compile,
    which cannot trace calls into a C library.)"""
    cfg = make_checkpoint(tmp_path, 128, seed=15)
    hf = G.load_quant(str(tmp_path), device="cuda", fuse_mlp=True, use_transformers=True)
    torch.manual_seed(5)
    prompt = torch.randint(1, cfg.vocab_size, (2, 8)).cuda()
    with torch.no_grad():
        a = hf.generate(prompt, max_new_tokens=6, do_sample=False, pad_token_id=0)
        b = hf.generate(prompt, max_new_tokens=6, do_sample=False, pad_token_id=0, cache_implementation="static", disable_compile=True)
    assert torch.equal(a, b)
