"""The reference's own verification grid and band (Verify.ipynb:96-139): groupsize in {-1, 128} x
M in {1, 8, 100, 256, 2048} x K, N in {4096, 11008}^2 on nn.Linear-initialised weights, round-to-nearest
quantised and packed (`dumbquant` + `pack_linear` there; quantize_rtn + pack_linear here), and the assertion
max |y - reference| <= 0.004 (Verify.ipynb:134).  The reference's yardstick is an fp16 nn.Linear on the
dequantised weights; here it is the float32 product of the oracle's dequantised weights with the fp16 input
(torch.matmul in float32 on the device - a library routine as the checker, the HIP path computes y)."""
import numpy as np
import pytest
import torch
import torch.nn as nn

import gptq_triton_amd as G
from oracle import gptq_oracle as O

pytestmark = pytest.mark.gpu

BAND = 0.004  # Verify.ipynb:134


@pytest.fixture(scope="module", params=[(4096, 4096), (4096, 11008), (11008, 4096), (11008, 11008)],
                ids=lambda kn: f"K{kn[0]}xN{kn[1]}")
def shape(request):
    return request.param


@pytest.mark.parametrize("groupsize", [-1, 128])
def test_reference_grid_within_the_reference_band(shape, groupsize):
    k, n = shape
    torch.manual_seed(0)
    layer = nn.Linear(k, n, bias=False)                       # default init, as in the notebook
    deq, scale, zero = G.quantize_rtn(layer.weight.data, groupsize)
    q = G.QuantLinear(4, groupsize, k, n, bias=False)
    G.pack_linear(q, deq, scale, zero)
    w16 = O.dequant_fp16(q.qweight.numpy(), q.qzeros.numpy(), q.scales.numpy(), groupsize)   # the oracle's weights [K, N]
    # the packed layer holds the quantiser's grid values up to the fp16 rounding of the scale
    assert np.abs(w16.astype(np.float32) - deq.t().numpy()).max() <= np.abs(deq).max().item() * 2.0 ** -9
    w32 = torch.from_numpy(w16).cuda().float()
    q = q.cuda()
    worst = 0.0
    for m in (1, 8, 100, 256, 2048):
        x = torch.randn((m, k), generator=torch.Generator().manual_seed(m)).half().cuda()
        y = q(x)
        ref = x.float() @ w32
        err = (y.float() - ref).abs().max().item()
        worst = max(worst, err)
        assert err <= BAND, f"K={k} N={n} g={groupsize} M={m}: max abs diff {err:.6f} above the reference's band"
        # and the band north_star states, elementwise
        assert bool(((y.float() - ref).abs() <= 2e-3 + 1e-2 * ref.abs()).all())
    print(f"K={k} N={n} g={groupsize}: worst max-abs diff over M = {worst:.6f}")
