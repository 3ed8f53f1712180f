"""The load-time quantiser against vectors written from the reference's own code
(tests/golden/make_rtn_vectors.py -> rtn_vectors.npz: Quantizer.find_params + quantize of gptq.py, driven per
group the way quantize.py's dumbquant drives them)."""
import os

import numpy as np
import pytest
import torch

import gptq_triton_amd as G

VECTORS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "rtn_vectors.npz")
CASES = ["gauss_g-1", "gauss_g128", "ties_g-1", "zero_group_g128", "nonneg_g128"]


@pytest.fixture(scope="module")
def vectors():
    return np.load(VECTORS)  # allow_pickle stays False


@pytest.mark.parametrize("name", CASES)
def test_rtn_quantiser_equals_the_reference_vectors(vectors, name):
    w = torch.from_numpy(vectors[name + "/weight"])
    g = int(vectors[name + "/groupsize"])
    deq, scale, zero = G.quantize_rtn(w, g, packable=False)
    # same float32 operations in the same order: equal bits, ties and the all-zero group included
    assert np.array_equal(scale.numpy(), vectors[name + "/scale"])
    assert np.array_equal(zero.numpy(), vectors[name + "/zero"])
    assert np.array_equal(deq.numpy(), vectors[name + "/deq"])


@pytest.mark.parametrize("name", CASES)
def test_packable_quantiser_differs_only_where_the_format_cannot_hold_the_zero_point(vectors, name):
    w = torch.from_numpy(vectors[name + "/weight"])
    g = int(vectors[name + "/groupsize"])
    gs = w.shape[1] if g == -1 else g
    deq, scale, zero = G.quantize_rtn(w, g)
    ref_zero, ref_scale, ref_deq = vectors[name + "/zero"], vectors[name + "/scale"], vectors[name + "/deq"]
    ok = ref_zero >= 1                       # [out, G]: groups the 4-bit stored zero (zero - 1) can hold
    assert np.array_equal(zero.numpy()[ok], ref_zero[ok]) and np.array_equal(scale.numpy()[ok], ref_scale[ok])
    ok_cols = np.repeat(ok, gs, axis=1)
    assert np.array_equal(deq.numpy()[ok_cols], ref_deq[ok_cols])
    assert (zero.numpy() >= 1).all() and (zero.numpy() <= 16).all()
    if name == "nonneg_g128":
        assert (~ok).any(), "the case is there to produce zero point 0 in the reference"
        # widened range: the largest weight of such a group stays on the grid, and nothing is clipped by more than half a step
        err = np.abs(deq.numpy() - w.numpy())
        assert (err <= np.repeat(scale.numpy(), gs, axis=1) * 0.5 + 1e-7).all()


def test_non_negative_group_round_trips_through_the_packer():
    from oracle import gptq_oracle as O
    rng = np.random.default_rng(5)
    w = torch.from_numpy(rng.random((256, 256)).astype(np.float32) * 0.05)   # [out, in], every group non-negative
    deq, scale, zero = G.quantize_rtn(w, 128)
    q = G.QuantLinear(4, 128, 256, 256, bias=False)
    G.pack_linear(q, deq, scale, zero)       # raised ValueError before: zero point 0 has no 4-bit stored form
    back = O.dequant_fp16(q.qweight.numpy(), q.qzeros.numpy(), q.scales.numpy(), 128).astype(np.float32)
    # the unpacked weights are the quantiser's grid values, up to the fp16 rounding of the scale
    assert np.abs(back - deq.t().numpy()).max() <= 0.05 * 2.0 ** -10
