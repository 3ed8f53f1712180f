"""gptq4_lm_head_argmax (decoder_ops.lm_head_argmax): the fp16 lm_head GEMV and the greedy argmax in one launch.
The logits are fp32 sums rounded to fp16 once; a library GEMV may round differently by an ulp, so on random data the
chosen index is checked against float64 logits (it must be within two fp16 ulps of the true maximum), and exactly on
data with a planted winner and on exact ties (the lower index wins, as torch.argmax)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def ops():
    from gptq_triton_amd import decoder_ops
    return decoder_ops


def head_is_zero():
    from gptq_triton_amd import _lib
    torch.cuda.synchronize()
    return all(int(ws[:_lib.WS_HEAD_BYTES].view(torch.int64).abs().sum()) == 0 for ws in _lib._workspaces.values())


@pytest.mark.parametrize("b,k,v", [(1, 4096, 32000), (8, 5120, 32000), (16, 4096, 32001), (3, 6656, 1000), (2, 8192, 5003), (1, 4096, 17)])
def test_against_float64_logits(b, k, v):
    rng = np.random.default_rng(b + k + v)
    x = rng.standard_normal((b, k)).astype(np.float16)
    w = (0.02 * rng.standard_normal((v, k))).astype(np.float16)
    out = ops().lm_head_argmax(torch.from_numpy(x).cuda().view(b, 1, k), torch.from_numpy(w).cuda(), max_rows=16)
    assert out.shape == (b, 1) and out.dtype == torch.int64
    logits = x.astype(np.float64) @ w.astype(np.float64).T
    got = out.cpu().numpy().reshape(b)
    for i in range(b):
        top = logits[i].max()
        assert 0 <= got[i] < v
        assert logits[i, got[i]] >= top - 2 * float(np.spacing(np.float16(abs(top)))), (i, got[i], int(logits[i].argmax()))
    assert head_is_zero()


def test_planted_winner_and_ties():
    rng = np.random.default_rng(5)
    b, k, v = 4, 4096, 32000
    x = rng.standard_normal((b, k)).astype(np.float16)
    w = (0.01 * rng.standard_normal((v, k))).astype(np.float16)
    winners = [31999, 0, 12345, 20000]
    for i, r in enumerate(winners):
        w[r] = (x[i].astype(np.float32) * 0.05).astype(np.float16)   # logit ~ 0.05 * |x|^2 = 200, far above the rest
    w[100] = w[20000]   # an exact tie for row 3: the lower index wins
    xd, wd = torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()
    out = ops().lm_head_argmax(xd, wd)
    assert out.tolist() == [31999, 0, 12345, 100]
    assert torch.equal(out, torch.nn.functional.linear(xd, wd).argmax(-1))
    # the same twice: nothing is left behind in the workspace
    assert torch.equal(ops().lm_head_argmax(xd, wd), out) and head_is_zero()


def test_other_shapes_go_through_torch():
    x = torch.randn(2, 1000, device="cuda").half()
    w = torch.randn(50, 1000, device="cuda").half()
    assert torch.equal(ops().lm_head_argmax(x, w), torch.nn.functional.linear(x, w).argmax(-1))
    from gptq_triton_amd import _lib
    lib = _lib.load()
    fake = 0x1000
    assert lib.gptq4_lm_head_argmax(fake, fake, fake, 1, 4000, 32000, fake, _lib.WS_HEAD_BYTES + (64 << 10), None) == -2
    assert lib.gptq4_lm_head_argmax(fake, fake, fake, 17, 4096, 32000, fake, _lib.WS_HEAD_BYTES + (64 << 10), None) == -2
    assert lib.gptq4_lm_head_argmax(fake, fake, fake, 1, 4096, 32000, fake, 64, None) == -4
    assert lib.gptq4_lm_head_argmax(None, fake, fake, 1, 4096, 32000, fake, _lib.WS_HEAD_BYTES + (64 << 10), None) == -1
