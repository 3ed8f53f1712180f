"""The two checkpoint-format conversions that also exist in plain torch, for a model that has been moved off the GPU
to be saved (act-order row sort; streaming order <-> checkpoint order), against the oracle's definitions, word for
word.  No GPU, no HIP library: these never touch the compute path."""
import numpy as np
import torch

from oracle import gptq_oracle as O


def _ql():
    from gptq_triton_amd import quant_linear
    return quant_linear


def test_sort_rows_on_the_cpu_moves_nibble_rows():
    ql = _ql()
    rng = np.random.default_rng(1)
    k, n = 256, 48
    q = rng.integers(0, 16, size=(k, n), dtype=np.uint8)
    perm = rng.permutation(k).astype(np.int32)
    qweight = O.pack_qweight(q)
    got = ql.sort_rows(torch.from_numpy(qweight), torch.from_numpy(perm))
    want = O.pack_qweight(q[perm])
    assert got.dtype == torch.int32 and got.shape == (k // 8, n)
    assert np.array_equal(got.numpy(), want)
    # and the inverse permutation puts the rows back
    inv = np.argsort(perm).astype(np.int32)
    back = ql.sort_rows(got, torch.from_numpy(inv))
    assert np.array_equal(back.numpy(), qweight)


def test_stream_pack_on_the_cpu_is_the_oracles_streaming_order():
    ql = _ql()
    for (k, n, g, seed) in ((1024, 256, 128, 2), (1024, 512, -1, 3), (2048, 256, 256, 4)):
        L = O.make_layer(k, n, g, seed=seed)
        sw, sm = ql.stream_pack(torch.from_numpy(L["qweight"]), torch.from_numpy(L["qzeros"]), torch.from_numpy(L["scales"]), g)
        ow, om = O.stream_order(L["qweight"], L["qzeros"], L["scales"])
        assert np.array_equal(sw.numpy(), ow), (k, n, g)
        assert np.array_equal(sm.numpy().reshape(-1), om.reshape(-1)), (k, n, g)
        # the word-by-word definition (loops) on the first shape only: it is slow
        if seed == 2:
            assert np.array_equal(sw.numpy(), O.stream_order_loops(L["qweight"]))
        back = ql.stream_unpack(sw)
        assert np.array_equal(back.numpy(), L["qweight"])
        assert np.array_equal(back.numpy(), O.unstream(ow))


def test_stream_pack_without_scales_gives_the_words_only():
    ql = _ql()
    L = O.make_layer(1024, 256, 128, seed=5)
    sw, sm = ql.stream_pack(torch.from_numpy(L["qweight"]))
    assert sm is None and np.array_equal(sw.numpy(), O.stream_order(L["qweight"])[0])
