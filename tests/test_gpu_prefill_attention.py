"""gptq4_prefill_attention through the C ABI (decoder_ops.prefill_attention): causal attention of a prompt, or of a
chunk behind cached tokens, against the float64 oracle - within the matmul tolerance of the path (|y - ref| <= 2e-3 +
1e-2 |ref|; the probabilities are rounded to fp16 before they meet V, as in torch's fused kernels) - and against
torch's own scaled_dot_product_attention on the same fp16 tensors."""
import numpy as np
import pytest
import torch

from oracle import gptq_oracle as O

pytestmark = pytest.mark.gpu


def ops():
    from gptq_triton_amd import decoder_ops
    return decoder_ops


def make(b, h, s, cap, seed, scale=1.0):
    rng = np.random.default_rng(seed)
    q = (scale * rng.standard_normal((b, h, s, 128))).astype(np.float16)
    k = (scale * rng.standard_normal((b, h, cap, 128))).astype(np.float16)
    v = rng.standard_normal((b, h, cap, 128)).astype(np.float16)
    return q, k, v


def close(got, ref, what):
    got = got.astype(np.float64)
    bad = np.abs(got - ref) > 2e-3 + 1e-2 * np.abs(ref)
    assert not bad.any(), f"{what}: {bad.sum()} of {bad.size} outside the tolerance, max abs {np.abs(got - ref).max():.3e}"


@pytest.mark.parametrize("b,h,s,cap,past", [(1, 2, 1, 1, 0), (2, 3, 5, 5, 0), (1, 4, 64, 64, 0), (1, 2, 65, 80, 0), (2, 2, 128, 128, 0),
                                            (1, 3, 300, 512, 0), (1, 2, 257, 700, 130), (2, 2, 100, 256, 64), (1, 2, 33, 400, 367),
                                            (1, 4, 1000, 1000, 0)])
def test_against_the_oracle(b, h, s, cap, past):
    q, k, v = make(b, h, s, cap, seed=s + past)
    # rows of the cache beyond past + s are never read: poison them
    k[:, :, past + s:] = np.nan
    v[:, :, past + s:] = np.nan
    out = ops().prefill_attention(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(), past)
    assert out.shape == (b, s, h * 128)
    close(out.cpu().numpy(), O.prefill_attention_ref(q, k, v, past), f"B={b} H={h} S={s} past={past}")


@pytest.mark.parametrize("b,h,s", [(1, 8, 300), (1, 13, 260), (5, 8, 140), (3, 25, 300), (8, 17, 129), (1, 80, 385)])
def test_every_head_and_query_block_of_many_heads(b, h, s):
    """Eight heads and more: a head's query blocks are dealt to one XCD (workgroup id % 8), the heads past the last multiple
    of eight separately, and more than eight heads to an XCD in groups of four - every (head, query block) exactly once."""
    q, k, v = make(b, h, s, s, seed=b * 1000 + h)
    out = ops().prefill_attention(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda())
    close(out.cpu().numpy(), O.prefill_attention_ref(q, k, v, 0), f"B={b} H={h} S={s}")


def test_peaked_scores_and_long_prompts():
    """Scores with a wide range (the running maximum moves a lot) at the benchmark's size: 2048 tokens."""
    b, h, s = 1, 4, 2048
    q, k, v = make(b, h, s, s, seed=3, scale=2.5)
    qd, kd, vd = (torch.from_numpy(a).cuda() for a in (q, k, v))
    out = ops().prefill_attention(qd, kd, vd)
    rows = np.array([0, 1, 31, 32, 63, 64, 127, 128, 129, 1000, 1023, 1024, 2046, 2047])
    ref = O.prefill_attention_ref(q, k, v, 0)[:, rows]
    close(out[:, rows].cpu().numpy(), ref, "peaked, S=2048")
    # torch's fused attention on the same tensors (fp16 in, fp32 inside): the same values within fp16 rounding of both
    t = torch.nn.functional.scaled_dot_product_attention(qd, kd, vd, is_causal=True).transpose(1, 2).reshape(b, s, h * 128)
    assert (out.float() - t.float()).abs().max().item() < 4e-3


def test_one_visible_key_returns_its_value_row_exactly():
    q, k, v = make(1, 2, 70, 70, seed=9)
    out = ops().prefill_attention(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda())
    assert np.array_equal(out[0, 0].cpu().numpy().reshape(2, 128), v[0, :, 0])


def test_argument_errors():
    from gptq_triton_amd import _lib
    lib = _lib.load()
    fake = 0x1000
    assert lib.gptq4_prefill_attention(None, fake, fake, fake, 1, 2, 8, 128, 8, 0, 1.0, None) == -1
    assert lib.gptq4_prefill_attention(fake, fake, fake, fake, 1, 2, 8, 64, 8, 0, 1.0, None) == -2
    assert lib.gptq4_prefill_attention(fake, fake, fake, fake, 1, 2, 8, 128, 8, 1, 1.0, None) == -2   # past + S beyond the cache
    assert lib.gptq4_prefill_attention(fake + 2, fake, fake, fake, 1, 2, 8, 128, 8, 0, 1.0, None) == -5
    with pytest.raises(RuntimeError):
        ops().prefill_attention(torch.zeros(1, 1, 4, 128, dtype=torch.float16), torch.zeros(1, 1, 4, 128, dtype=torch.float16),
                                torch.zeros(1, 1, 4, 128, dtype=torch.float16))
