"""GPU test of gptq4_matmul_static, the entry point for callers that cannot allocate device memory: called
through the C ABI, its output equals gptq4_matmul's (same kernels, same launch plans, hence the same
bits) on two calls in a row - the second with a smaller input, so that whatever the first call left in the
library's scratch array is in the way of the second if it is not handled - and the oracle's values within the
stated tolerance.  Calls beyond the array's size are rejected on the host."""
import numpy as np
import pytest
import torch

from conftest import to_dev
from oracle import gptq_oracle as O

pytestmark = pytest.mark.gpu

TOL_ABS, TOL_REL = 2e-3, 1e-2  # |y - y_ref| <= 2e-3 + 1e-2 * |y_ref|


def _both(lib, x, D, k, n, g, bias=None):
    from gptq_triton_amd import _lib
    m = x.shape[0]
    stream = _lib.current_stream(x.device)
    y_ws = torch.empty((m, n), dtype=torch.float16, device=x.device)
    y_st = torch.full((m, n), float("nan"), dtype=torch.float16, device=x.device)
    need = lib.gptq4_workspace_bytes(_lib.OP_MATMUL, m, k, n)
    ws = torch.zeros(need, dtype=torch.uint8, device=x.device)
    rc = lib.gptq4_matmul(x.data_ptr(), D["qweight"].data_ptr(), D["qzeros"].data_ptr(), D["scales"].data_ptr(), None,
                          _lib.ptr(bias), y_ws.data_ptr(), m, k, n, g, ws.data_ptr(), ws.numel(), stream)
    assert rc == 0, lib.gptq4_strerror(rc)
    rc = lib.gptq4_matmul_static(x.data_ptr(), D["qweight"].data_ptr(), D["qzeros"].data_ptr(), D["scales"].data_ptr(),
                                 _lib.ptr(bias), y_st.data_ptr(), m, k, n, g, stream)
    assert rc == 0, lib.gptq4_strerror(rc)
    torch.cuda.synchronize()
    return y_ws, y_st


def test_static_scratch_matmul_equals_workspace_matmul_twice_in_a_row():
    from gptq_triton_amd import _lib
    lib = _lib.load()
    # first call: 16 rows, split-K across workgroups (partial sums and counters in the scratch array);
    # second call: fewer rows of a smaller matrix, other tile and split counts
    for (m, k, n, g, seed) in ((16, 4096, 4096, 128, 11), (3, 1024, 2048, -1, 12), (1, 4096, 4096, 128, 13)):
        L = O.make_layer(k, n, g, seed=seed)
        D = to_dev(L)
        x = O.make_x(m, k, seed=seed + 100)
        xd = torch.from_numpy(x).cuda()
        y_ws, y_st = _both(lib, xd, D, k, n, g)
        assert torch.equal(y_ws, y_st), f"M={m} K={k} N={n}: static-scratch result differs from the workspace call"
        ref = O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g)
        got = y_st.cpu().numpy().astype(np.float64)
        assert (np.abs(got - ref) <= TOL_ABS + TOL_REL * np.abs(ref)).all(), f"M={m} K={k} N={n}: outside the tolerance"


def test_static_scratch_takes_mid_sized_calls_and_bias():
    from gptq_triton_amd import _lib
    lib = _lib.load()
    m, k, n, g = 48, 1024, 1024, 128
    L = O.make_layer(k, n, g, seed=21)
    D = to_dev(L)
    x = torch.from_numpy(O.make_x(m, k, seed=22)).cuda()
    bias = torch.from_numpy(np.random.default_rng(3).standard_normal(n).astype(np.float16)).cuda()
    y_ws, y_st = _both(lib, x, D, k, n, g, bias)
    assert torch.equal(y_ws, y_st)
    # and one decode-sized call right after it
    x1 = torch.from_numpy(O.make_x(2, k, seed=23)).cuda()
    y_ws, y_st = _both(lib, x1, D, k, n, g, bias)
    assert torch.equal(y_ws, y_st)


def test_static_scratch_rejects_what_does_not_fit():
    from gptq_triton_amd import _lib
    lib = _lib.load()
    fake = 0x1000  # never dereferenced: rejected on the host
    # 16 rows of 32768 columns would need 32 MiB of partial sums
    assert lib.gptq4_workspace_bytes(_lib.OP_MATMUL, 16, 4096, 32768) > _lib.STATIC_SCRATCH_BYTES
    assert lib.gptq4_matmul_static(fake, fake, fake, fake, None, fake, 16, 4096, 32768, -1, None) == -6
    assert b"scratch" in lib.gptq4_strerror(-6)
    # the ordinary argument errors come first
    assert lib.gptq4_matmul_static(None, fake, fake, fake, None, fake, 1, 4096, 4096, -1, None) == -1
    assert lib.gptq4_matmul_static(fake, fake, fake, fake, None, fake, 1, 4000, 4096, -1, None) == -2


def test_static_scratch_status_and_reset():
    """The library's array is private: gptq4_static_status reports a bounded wait that ran out (forced from the
    host with the spin-limit hook; every kernel exits normally), gptq4_static_reset zeroes the head, and the next
    call is right again."""
    from gptq_triton_amd import _lib
    lib = _lib.load()
    m, k, n, g = 1, 4096, 4096, 128
    L = O.make_layer(k, n, g, seed=31)
    D = to_dev(L)
    xd = torch.from_numpy(O.make_x(m, k, seed=32)).cuda()
    stream = _lib.current_stream(xd.device)
    y = torch.empty((m, n), dtype=torch.float16, device="cuda")

    def call():
        return lib.gptq4_matmul_static(xd.data_ptr(), D["qweight"].data_ptr(), D["qzeros"].data_ptr(), D["scales"].data_ptr(),
                                       None, y.data_ptr(), m, k, n, g, stream)

    assert call() == 0 and lib.gptq4_static_status(stream) == 0
    try:
        lib.gptq4_set_exchange_spin_limit(0xFFFFFFFF)
        assert call() == 0
        assert lib.gptq4_static_status(stream) == -7
        assert b"wait" in lib.gptq4_strerror(-7)
    finally:
        lib.gptq4_set_exchange_spin_limit(0)
        torch.cuda.synchronize()
        assert lib.gptq4_static_reset(stream) == 0
    assert lib.gptq4_static_status(stream) == 0
    y_ws, y_st = _both(lib, xd, D, k, n, g)
    assert torch.equal(y_ws, y_st)
