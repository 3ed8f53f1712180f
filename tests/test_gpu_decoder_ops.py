"""GPU parity of the decoder-side kernels (RMSNorm, single-query attention over the KV
cache) against the oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from conftest import bits
from oracle import gptq_oracle as O

pytestmark = pytest.mark.gpu


def gptq():
    import gptq_triton_amd
    return gptq_triton_amd


@pytest.mark.parametrize("m,h", [(1, 4096), (3, 5120), (17, 6656), (2048, 4096), (5, 64), (2, 8200)])
def test_rmsnorm(m, h):
    rng = np.random.default_rng(m + h)
    x = (rng.standard_normal((m, h)) * rng.uniform(0.01, 30.0, size=(m, 1))).astype(np.float16)
    w = (1.0 + 0.1 * rng.standard_normal(h)).astype(np.float16)
    y = gptq().rms_norm(torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda(), 1e-6).cpu().numpy()
    ref = O.rmsnorm_ref(x, w, 1e-6)
    # fp32 statistics against float64: the normalised value can round one fp16 step apart
    diff = np.abs(y.astype(np.float64) - ref.astype(np.float64))
    assert (diff <= 2 * np.spacing(np.abs(ref)).astype(np.float64)).all()
    assert (bits(y) == bits(ref)).mean() > 0.98


@pytest.mark.parametrize("m,h", [(1, 4096), (4, 5120), (300, 6656), (2, 8200)])
def test_add_rmsnorm(m, h):
    rng = np.random.default_rng(m * h)
    x = (rng.standard_normal((m, h)) * 3).astype(np.float16)
    d = rng.standard_normal((m, h)).astype(np.float16)
    w = (1.0 + 0.1 * rng.standard_normal(h)).astype(np.float16)
    s, y = gptq().add_rms_norm(torch.from_numpy(x).cuda(), torch.from_numpy(d).cuda(), torch.from_numpy(w).cuda(), 1e-6)
    s_ref = (x + d).astype(np.float16)   # one fp16 add, as torch does
    assert np.array_equal(bits(s.cpu().numpy()), bits(s_ref))
    ref = O.rmsnorm_ref(s_ref, w, 1e-6)
    diff = np.abs(y.cpu().numpy().astype(np.float64) - ref.astype(np.float64))
    assert (diff <= 2 * np.spacing(np.abs(ref)).astype(np.float64)).all()
    # and it is the unfused kernel applied to the sum, bit for bit
    y2 = gptq().rms_norm(s, torch.from_numpy(w).cuda(), 1e-6)
    assert torch.equal(y, y2)


@pytest.mark.parametrize("m,h", [(1, 4096), (8, 5120), (16, 13824), (40, 6656), (2, 8200)])
def test_norms_store_in_a_given_order(m, h):
    """With out_index, value f of every row lands at position out_index[f]: the same bits, moved (rows longer
    than the 8192 values held in registers included); the sum keeps its order."""
    G = gptq()
    gen = torch.Generator(device="cuda"); gen.manual_seed(m + h)
    x = (3 * torch.randn((m, h), device="cuda", generator=gen)).half()
    d = torch.randn((m, h), device="cuda", generator=gen).half()
    w = (1 + 0.1 * torch.randn(h, device="cuda", generator=gen)).half()
    order = torch.randperm(h, device="cuda", generator=gen).int()
    y = G.rms_norm(x, w, 1e-6)
    moved = G.rms_norm(x, w, 1e-6, out_index=order)
    want = torch.empty_like(y)
    want[:, order.long()] = y
    assert torch.equal(moved, want)
    s, y = G.add_rms_norm(x, d, w, 1e-6)
    s2, moved = G.add_rms_norm(x, d, w, 1e-6, out_index=order)
    want[:, order.long()] = y
    assert torch.equal(s, s2) and torch.equal(moved, want)
    # the moved values may not land in a tensor that is still being read
    from gptq_triton_amd import _lib
    lib = _lib.load()
    stream = _lib.current_stream(x.device)
    rc = lib.gptq4_rmsnorm(x.data_ptr(), w.data_ptr(), x.data_ptr(), order.data_ptr(), m, h, 1e-6, stream)
    assert rc < 0 and b"shape" in lib.gptq4_strerror(rc).lower()
    rc = lib.gptq4_add_rmsnorm(x.data_ptr(), d.data_ptr(), w.data_ptr(), s.data_ptr(), d.data_ptr(), order.data_ptr(), m, h, 1e-6,
                               stream)
    assert rc < 0


def test_rmsnorm_keeps_batch_dims_and_rejects_host_tensors():
    x = torch.randn(2, 3, 256).half()
    w = torch.ones(256).half()
    with pytest.raises(RuntimeError):
        gptq().rms_norm(x, w, 1e-6)
    y = gptq().rms_norm(x.cuda(), w.cuda(), 1e-6)
    assert y.shape == (2, 3, 256)
    assert np.array_equal(y.cpu().numpy(), O.rmsnorm_ref(x.numpy(), w.numpy(), 1e-6)) or \
        (np.abs(y.cpu().numpy().astype(np.float32) - O.rmsnorm_ref(x.numpy(), w.numpy(), 1e-6).astype(np.float32)) < 4e-3).all()


@pytest.mark.parametrize("bsz,heads,cap,positions", [(1, 32, 2176, [2047]), (2, 8, 40, [0, 39]), (3, 5, 300, [1, 150, 299]),
                                                     (8, 52, 515, [3, 100, 200, 300, 400, 500, 514, 64]), (1, 2, 16, [15])])
def test_decode_attention(bsz, heads, cap, positions):
    rng = np.random.default_rng(cap + heads)
    q = rng.standard_normal((bsz, heads, 1, 128)).astype(np.float16)
    k = rng.standard_normal((bsz, heads, cap, 128)).astype(np.float16)
    v = rng.standard_normal((bsz, heads, cap, 128)).astype(np.float16)
    pos = np.asarray(positions, dtype=np.int32)
    # rows beyond each position hold poison: they must not be read into the result
    for b, p in enumerate(positions):
        k[b, :, p + 1:] = 300.0
        v[b, :, p + 1:] = -1000.0
    out = gptq().decode_attention(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(),
                                  torch.from_numpy(pos).cuda())
    assert out.shape == (bsz, 1, heads * 128) and out.dtype == torch.float16
    ref = O.decode_attention_ref(q, k, v, positions)
    err = np.abs(out.cpu().numpy().astype(np.float64) - ref)
    assert (err <= 2e-3 + 1e-2 * np.abs(ref)).all(), err.max()
    assert err.max() < 2e-3  # fp32 softmax of fp16 inputs, one fp16 rounding of the result
    # with an output order, feature f of every row lands at position order[f]: same values, moved
    order = torch.from_numpy(np.random.default_rng(1).permutation(heads * 128).astype(np.int32)).cuda()
    moved = gptq().decode_attention(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(),
                                    torch.from_numpy(pos).cuda(), out_index=order)
    want = torch.empty_like(out)
    want[..., order.long()] = out
    assert torch.equal(moved, want)


def test_decode_attention_peaked_scores_do_not_overflow():
    q = torch.zeros(1, 1, 1, 128).half(); q[..., :] = 30.0
    k = torch.zeros(1, 1, 70, 128).half(); k[0, 0, 33] = 30.0; k[0, 0, 2] = -30.0
    v = torch.randn(1, 1, 70, 128).half()
    out = gptq().decode_attention(q.cuda(), k.cuda(), v.cuda(), torch.tensor([69], dtype=torch.int32).cuda())
    assert torch.isfinite(out).all()
    assert torch.equal(out.cpu().reshape(128), v[0, 0, 33])
