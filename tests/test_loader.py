"""Checkpoint format: packer, save/load round trip, model surgery by load_quant (CPU), and
the loaded model on the GPU against a float32 CPU reference decoder."""
import json
import os

import numpy as np
import pytest
import torch
import torch.nn as nn

import gptq_triton_amd as G
from gptq_triton_amd.llama import LlamaForCausalLM
from oracle import gptq_oracle as O


def tiny_config(**kw):
    cfg = G.LlamaConfigLite(hidden_size=256, num_attention_heads=2, max_position_embeddings=512,
                            intermediate_size=768, num_hidden_layers=2, vocab_size=320)
    for k, v in kw.items():
        setattr(cfg, k, v)
    return cfg


def make_checkpoint(path, groupsize, safetensors=True, seed=0, act_order=False):
    """Random fp16 model -> RTN-quantised, packed, saved in the reference layout."""
    torch.manual_seed(seed)
    cfg = tiny_config()
    model = LlamaForCausalLM(cfg).half()
    for p in model.parameters():
        p.requires_grad_(False)
    model.model.embed_tokens.weight.normal_(0, 1.0)
    for n, m in model.named_modules():
        if isinstance(m, nn.Linear):
            m.weight.normal_(0, 0.05)
    floats = {n: m.weight.clone() for n, m in model.named_modules() if isinstance(m, nn.Linear) and n != "lm_head"}
    G.make_quant(model, 4, groupsize, act_order=act_order)
    gen = torch.Generator().manual_seed(seed + 1)
    shared = {}
    for n, m in model.named_modules():
        if isinstance(m, G.QuantLinear):
            deq, scale, zero = G.quantize_rtn(floats[n], groupsize)
            G.pack_linear(m, deq, scale, zero)
            if act_order:
                # q/k/v (and gate/up) share their input, hence one g_idx per group of projections
                key = (n.rsplit(".", 1)[0], m.infeatures, n.endswith(("o_proj", "down_proj")))
                if key not in shared:
                    shared[key] = torch.randperm(m.infeatures, generator=gen)
                perm = shared[key]
                # scatter the rows so that row r of the new layout is old row perm[r]
                q = torch.from_numpy(O.unpack_qweight(m.qweight.numpy()))[perm]
                m.qweight = torch.from_numpy(O.pack_qweight(q.numpy()))
                m.g_idx = (perm // m.groupsize).to(torch.int32)
    G.save_quant(model, path, 4, groupsize, safetensors=safetensors)
    return cfg


def test_packer_layout_and_round_trip():
    torch.manual_seed(3)
    w = torch.randn(256, 512) * 0.1          # [out, in]
    for gs in (-1, 128):
        deq, scale, zero = G.quantize_rtn(w, gs)
        ql = G.QuantLinear(4, gs, 512, 256, bias=False)
        G.pack_linear(ql, deq, scale, zero)
        # integer weights recomputed independently, then the oracle's unpackers
        g = 512 if gs == -1 else gs
        q_expect = torch.round(w.reshape(256, 512 // g, g) / scale[..., None]).add(zero[..., None]).clamp(0, 15)
        q_expect = q_expect.reshape(256, 512).t().numpy().astype(np.uint8)
        assert (O.unpack_qweight(ql.qweight.numpy()) == q_expect).all()
        assert (O.unpack_qzeros(ql.qzeros.numpy()) == (zero.t().numpy() - 1).astype(np.uint8)).all()
        assert ql.qweight.dtype == torch.int32 and ql.qweight.shape == (64, 256)
        # decoding gives back the grid values up to the fp16 rounding of scale and weight
        W = O.dequant_fp16(ql.qweight.numpy(), ql.qzeros.numpy(), ql.scales.numpy(), gs)
        assert np.abs(W.astype(np.float32) - deq.t().numpy()).max() < 2e-3
        # quantisation error itself is at most half a step
        assert (deq - w).abs().max() <= scale.max() / 2 + 1e-6
    # the first eight input rows of column 0 are the eight nibbles of word (0, 0), LSB first
    ql = G.QuantLinear(4, -1, 128, 256, bias=False)
    wq = torch.zeros(256, 128)
    wq[0, :8] = torch.arange(8).float()
    G.pack_linear(ql, wq, torch.ones(256, 1), torch.ones(256, 1))      # scale 1, zero 1: q = w + 1
    assert int(ql.qweight[0, 0]) & 0xFFFFFFFF == 0x87654321
    assert int(ql.qzeros[0, 0]) == 0                                    # stored zero = true zero - 1
    with pytest.raises(ValueError):
        G.pack_linear(ql, wq + 100, torch.ones(256, 1), torch.ones(256, 1))


@pytest.mark.parametrize("groupsize,safetensors", [(-1, True), (128, True), (128, False)])
def test_load_quant_surgery_on_cpu(tmp_path, groupsize, safetensors):
    cfg = make_checkpoint(tmp_path, groupsize, safetensors)
    assert os.path.exists(tmp_path / ("model.safetensors" if safetensors else "model.pt"))
    assert json.load(open(tmp_path / "quant_config.json")) == {"wbits": 4, "groupsize": groupsize}
    model = G.load_quant(str(tmp_path), warmup_autotune=False, device=None)
    attn = model.model.layers[1].self_attn
    assert isinstance(attn, G.QuantLlamaAttention)
    assert attn.qkv_proj.qweight.shape == (256 // 8, 3 * 256) and isinstance(attn.o_proj, G.QuantLinear)
    mlp = model.model.layers[0].mlp
    # the reference fuses the MLP by default only without grouping (__init__.py:76-77)
    assert isinstance(mlp, G.QuantLlamaMLP) == (groupsize == -1)
    assert isinstance(model.lm_head, nn.Linear) and model.lm_head.weight.dtype == torch.float16
    assert model.seqlen == 2048
    fused = G.load_quant(str(tmp_path), warmup_autotune=False, device=None, fuse_mlp=True)
    assert isinstance(fused.model.layers[0].mlp, G.QuantLlamaMLP)
    # fused QKV tensors are the three projections side by side, q then k then v
    from safetensors.torch import load_file
    state = load_file(str(tmp_path / "model.safetensors")) if safetensors else torch.load(tmp_path / "model.pt", weights_only=True)
    cat = torch.cat([state[f"model.layers.1.self_attn.{n}_proj.qweight"] for n in "qkv"], dim=1)
    assert torch.equal(attn.qkv_proj.qweight, cat)


def test_load_quant_errors(tmp_path):
    make_checkpoint(tmp_path, -1)
    with pytest.raises(ValueError, match="device"):
        G.load_quant(str(tmp_path), warmup_autotune=True, device=None)
    os.remove(tmp_path / "model.safetensors")
    with pytest.raises(FileNotFoundError):
        G.load_quant(str(tmp_path), warmup_autotune=False, device=None)


def test_all_zero_bias_is_dropped(tmp_path):
    cfg = make_checkpoint(tmp_path, -1)
    from safetensors.torch import load_file, save_file
    state = load_file(str(tmp_path / "model.safetensors"))
    state["model.layers.0.self_attn.o_proj.bias"] = torch.zeros(256, dtype=torch.float16)
    save_file(state, str(tmp_path / "model.safetensors"))
    # a checkpoint with a bias tensor needs a bias buffer: build the skeleton by hand as the loader does
    model = G.load_quant(str(tmp_path), warmup_autotune=False, device=None)
    assert model.model.layers[0].self_attn.o_proj.bias is None


@pytest.mark.gpu
@pytest.mark.parametrize("groupsize,act_order", [(-1, False), (128, False), (128, True)])
def test_loaded_model_matches_cpu_reference(tmp_path, groupsize, act_order):
    from oracle import decoder_ref
    from safetensors.torch import load_file
    cfg = make_checkpoint(tmp_path, groupsize, act_order=act_order, seed=7)
    state = load_file(str(tmp_path / "model.safetensors"))
    model = G.load_quant(str(tmp_path), device="cuda", fuse_mlp=True)
    torch.manual_seed(1)
    ids = torch.randint(0, cfg.vocab_size, (2, 40))
    ref = decoder_ref.forward(state, cfg, groupsize, ids)
    logits, _ = model(ids.cuda())
    got = logits.float().cpu()
    # fp16 activations through 2 layers against a float32 reference.  Measured over 9 such checkpoints (3 seeds x
    # 3 configurations): logits up to 4.5 in magnitude, largest error 0.0021-0.0026, mean error 4.0e-4 - about two
    # fp16 roundings of the hidden state.  The bound is 2.3 times the largest error seen; where the reference's
    # best logit leads by more than twice the bound, the greedy token must be the same.
    bound = 0.006
    err = (got - ref).abs()
    assert err.max().item() < bound and err.mean().item() < 1e-3, (err.max().item(), err.mean().item())
    top2 = ref.topk(2, dim=-1).values
    clear = (top2[..., 0] - top2[..., 1]) > 2 * bound
    assert clear.float().mean() > 0.8, "the check needs positions with a clear winner"
    assert torch.equal(got.argmax(-1)[clear], ref.argmax(-1)[clear])

    # incremental decoding with the KV cache equals the full forward
    full, _ = model(ids.cuda())
    part, past = model(ids[:, :30].cuda(), use_cache=True)
    steps = [part]
    for t in range(30, 40):
        lg, past = model(ids[:, t:t + 1].cuda(), past_key_values=past, use_cache=True)
        steps.append(lg)
    inc = torch.cat(steps, dim=1)
    assert (inc.float() - full.float()).abs().max() < 0.03 * full.float().abs().max()

    # greedy generation with the preallocated cache follows the argmax of the full forward
    out = model.generate_greedy(ids[:, :8].cuda(), 6)
    assert out.shape == (2, 14) and torch.equal(out[:, :8].cpu(), ids[:, :8])
    cur = ids[:, :8].cuda()
    for _ in range(6):
        lg, _ = model(cur)
        cur = torch.cat([cur, lg[:, -1:].argmax(-1)], dim=1)
    assert (out == cur).float().mean() > 0.9


@pytest.mark.gpu
@pytest.mark.parametrize("groupsize,act_order,bsz", [(128, False, 1), (128, True, 3), (-1, False, 2)])
def test_graph_replayed_decode_equals_eager_decode(tmp_path, groupsize, act_order, bsz):
    """The captured decode step (K/V placed by position id, attention over the whole cache
    under a position mask) gives the tokens of the step launched kernel by kernel, on
    every replay."""
    cfg = make_checkpoint(tmp_path, groupsize, act_order=act_order, seed=11)
    model = G.load_quant(str(tmp_path), device="cuda", fuse_mlp=True)
    torch.manual_seed(3)
    ids = torch.randint(0, cfg.vocab_size, (bsz, 9)).cuda()
    eager = model.generate_greedy(ids, 12)
    graph = model.generate_greedy(ids, 12, use_graph=True)
    assert eager.shape == (bsz, 21)
    assert torch.equal(eager, graph)
    # a decoder can be prefilled again and its graph replayed with other contents
    from gptq_triton_amd.llama import GreedyDecoder
    dec = GreedyDecoder(model, bsz, 32)
    for seed in (4, 5):
        torch.manual_seed(seed)
        ids2 = torch.randint(0, cfg.vocab_size, (bsz, 7)).cuda()
        first = dec.prefill(ids2)
        rest = dec.decode(10, use_graph=True)
        want = model.generate_greedy(ids2, 11)
        assert torch.equal(torch.cat([ids2, first, rest], dim=1), want)
    # and the decoder's tokens are those of the module-by-module forward over the growing sequence (which has
    # neither the decoder's cache placement by position nor its attention output in o_proj's row order)
    cur = ids
    for _ in range(12):
        lg, _ = model(cur)
        cur = torch.cat([cur, lg[:, -1:].argmax(-1)], dim=1)
    assert (eager == cur).float().mean() > 0.9


@pytest.mark.gpu
def test_qkv_rotary_places_kv_by_position():
    import numpy as np
    from conftest import to_dev
    from oracle import gptq_oracle as O
    from gptq_triton_amd.fused_attention import KV_AT_POSITION
    H, Dh, hidden, g, cap = 8, 128, 1024, 128, 24
    L = O.make_layer(hidden, 3 * hidden, g, seed=300)
    D = to_dev(L)
    cos, sin = G.RotaryTable(Dh, 2048).get(torch.device("cuda"), 2048)
    for s in (1, 5, 20):   # 20 rows of 2 sequences: the tiled kernel
        x = O.make_x(2 * s, hidden, seed=301 + s).reshape(2, s, hidden)
        pos = np.stack([np.arange(s) + 2, np.arange(s)[::-1].copy() + 1]).astype(np.int32)
        kc = torch.full((2, H, cap, Dh), 7.0, dtype=torch.float16, device="cuda")
        vc = torch.full((2, H, cap, Dh), 7.0, dtype=torch.float16, device="cuda")
        xd, pd = torch.from_numpy(x).cuda(), torch.from_numpy(pos).cuda()
        q, _, _ = G.qkv_rotary(g, xd, D["qweight"], D["scales"], D["qzeros"], pd, cos, sin, H, Dh,
                               kv_out=(kc, vc), kv_offset=KV_AT_POSITION)
        q0, k0, v0 = G.qkv_rotary(g, xd, D["qweight"], D["scales"], D["qzeros"], pd, cos, sin, H, Dh)
        assert torch.equal(q, q0)
        for b in range(2):
            rows = torch.from_numpy(pos[b].astype(np.int64)).cuda()
            assert torch.equal(kc[b][:, rows], k0[b]) and torch.equal(vc[b][:, rows], v0[b])
            untouched = torch.ones(cap, dtype=torch.bool)
            untouched[pos[b]] = False
            assert bool((kc[b][:, untouched] == 7.0).all()) and bool((vc[b][:, untouched] == 7.0).all())


@pytest.mark.gpu
@pytest.mark.parametrize("use_graph", [False, True])
def test_decode_past_max_position_embeddings_keeps_rotating(tmp_path, use_graph):
    """A decode step places K/V by the position buffer on the device; the rotary table it reads must cover the
    whole cache, not just config.max_position_embeddings (positions beyond the table are clamped to its last
    row, which silently freezes the rotation).  The cache rows written by 11 decode steps past the 16 positions
    of the config equal those of one forward pass over the whole sequence."""
    from gptq_triton_amd.llama import GreedyDecoder
    torch.manual_seed(13)
    cfg = make_checkpoint(tmp_path, 128, seed=13)
    model = G.load_quant(str(tmp_path), device="cuda", fuse_mlp=True)
    for layer in model.model.layers:          # a table of 16 rows unless the call asks for more
        layer.self_attn.max_position_embeddings = 16
        layer.self_attn.rope = G.RotaryTable(layer.self_attn.head_dim, 16)
    ids = torch.randint(0, cfg.vocab_size, (2, 9)).cuda()
    dec = GreedyDecoder(model, 2, 9 + 12)
    first = dec.prefill(ids)
    rest = dec.decode(11, use_graph=use_graph)
    seq = torch.cat([ids, first, rest], dim=1)            # 21 tokens; the cache holds the first 20
    _, past = model(seq[:, :20], use_cache=True)
    for (kc, vc), (k_full, v_full) in zip(dec.caches, past):
        assert (kc[:, :, :20].float() - k_full.float()).abs().max().item() < 0.03 * k_full.float().abs().max().item()
        assert (vc[:, :, :20].float() - v_full.float()).abs().max().item() < 0.03 * v_full.float().abs().max().item()


@pytest.mark.gpu
@pytest.mark.parametrize("fuse_mlp", [True, False])
def test_compacted_act_order_model_keeps_one_copy_and_the_checkpoint_layout_outside(tmp_path, fuse_mlp):
    """load_quant(compact=True), the default: an act-order model on the GPU holds each packed weight once, in the
    layout the kernels read.  Same logits bit for bit as the uncompacted model, state_dict() / save_quant() give the
    checkpoint's tensors, and load_state_dict() of other weights is followed."""
    from safetensors.torch import load_file
    cfg = make_checkpoint(tmp_path / "a", 128, act_order=True, seed=21)
    make_checkpoint(tmp_path / "b", 128, act_order=True, seed=22)
    state_a = load_file(str(tmp_path / "a" / "model.safetensors"))
    plain = G.load_quant(str(tmp_path / "a"), device="cuda", fuse_mlp=fuse_mlp, compact=False)
    compact = G.load_quant(str(tmp_path / "a"), device="cuda", fuse_mlp=fuse_mlp)
    ids = torch.randint(0, cfg.vocab_size, (2, 24), generator=torch.Generator().manual_seed(4)).cuda()
    want, _ = plain(ids)
    got, _ = compact(ids)
    assert torch.equal(got, want)

    # one copy: no derived copies beside the buffers, and the buffers are not the checkpoint layout
    attn, mlp = compact.model.layers[0].self_attn, compact.model.layers[0].mlp
    assert attn.o_proj._sorted is None and attn.o_proj._compact_perm is not None
    assert not torch.equal(attn.o_proj.qweight.cpu(), state_a["model.layers.0.self_attn.o_proj.qweight"])
    assert torch.equal(attn.o_proj.checkpoint_qweight().cpu(), state_a["model.layers.0.self_attn.o_proj.qweight"])
    if fuse_mlp:
        assert mlp._is_compact and mlp._sorted is None and mlp._chained is None
        x = torch.randn(3, cfg.hidden_size, device="cuda").half()
        assert torch.equal(mlp.gate_up(x), plain.model.layers[0].mlp.gate_up(x))

    # the checkpoint layout on the way out: the same tensors as the uncompacted model's state_dict
    sd_plain, sd_compact = plain.state_dict(), compact.state_dict()
    assert sd_plain.keys() == sd_compact.keys()
    for key in sd_plain:
        assert torch.equal(sd_plain[key], sd_compact[key]), key
    # dequantised weights too
    assert torch.equal(attn.o_proj.dequantize(), plain.model.layers[0].self_attn.o_proj.dequantize())

    # other weights loaded into the compacted model: back to the checkpoint layout, then the new model's logits
    other = G.load_quant(str(tmp_path / "b"), device="cuda", fuse_mlp=fuse_mlp, compact=False)
    compact.load_state_dict(other.state_dict())
    assert compact.model.layers[0].self_attn.o_proj._compact_perm is None
    want_b, _ = other(ids)
    got_b, _ = compact(ids)
    assert torch.equal(got_b, want_b) and not torch.equal(got_b, want)
    # and compacting again by hand
    G.quant_linear.compact_act_order(compact)
    again, _ = compact(ids)
    assert torch.equal(again, want_b)
