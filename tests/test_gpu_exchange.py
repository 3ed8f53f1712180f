"""GPU tests of the two ways workgroups of the small-M kernels hand over partial sums: plain sums under an arrival
counter (the last to arrive finishes the tile) and marked 8-byte values (a fixed finisher polls for them).  Both
must give the oracle's result, bit-identical to each other (the sums are added in split order either way), leave the
head of the workspace zero, and the bounded wait of the second must end a call - with the error word set - when its
limit is hit."""
import numpy as np
import pytest
import torch

from conftest import to_dev
from oracle import gptq_oracle as O
from test_gpu_parity import assert_close, gptq

pytestmark = pytest.mark.gpu

COUNTERS, MARKED = 10, 20   # added to the load width of gptq4_set_tuning


@pytest.fixture
def split_k_only():
    """The balanced GEMV off, so that every call reaches the split-K kernel."""
    from gptq_triton_amd import _lib
    lib = _lib.load()
    lib.gptq4_set_gemv_tuning(0, 0, 0, 0)
    yield lib
    lib.gptq4_set_tuning(0, 0, 0)
    lib.gptq4_set_gemv_tuning(1, 0, 0, 0)


def _head_is_zero(device):
    from gptq_triton_amd import _lib
    ws = _lib.workspace(device, 0)
    torch.cuda.synchronize()
    return int(ws[:_lib.WS_HEAD_BYTES].view(torch.int32).abs().sum()) == 0


@pytest.mark.parametrize("words", [1, 2, 4])
@pytest.mark.parametrize("splitk", [2, 5, 8, 16])
@pytest.mark.parametrize("m", [1, 4, 16])
def test_both_exchanges_give_the_oracle_result_bit_identically(split_k_only, words, splitk, m):
    lib = split_k_only
    G = gptq()
    n, g = 768, 128
    k = 8192 if splitk == 16 else 2048       # 64 K batches of 128: every wave of 16 splits has one; else 16 batches
    heads = k // 128
    gate = O.make_layer(k, n, g, seed=60 + words, bias=True)
    up = O.make_layer(k, n, g, seed=61 + words)
    qkv = O.make_layer(k, 3 * k, g, seed=62) if k == 2048 else None
    x = O.make_x(m, k, seed=63 + m)
    xd = torch.from_numpy(x).cuda()
    Dg, Du = to_dev(gate), to_dev(up)
    Dq = to_dev(qkv) if qkv is not None else None
    cos, sin = G.RotaryTable(128, 64).get(torch.device("cuda"), 64)
    pos = (np.arange(m) % 50)[:, None].astype(np.int32)
    got = {}
    for mode in (COUNTERS, MARKED):
        lib.gptq4_set_tuning(mode + words, 0, splitk)
        y = G.matmul4(g, xd, Dg["qweight"], Dg["scales"], Dg["qzeros"], Dg["bias"])
        h = G.llama_mlp_4(g, xd, Dg["qweight"], Dg["scales"], Dg["qzeros"], Du["qweight"], Du["scales"], Du["qzeros"])
        r = None
        if Dq is not None:
            r = G.qkv_rotary(g, xd.view(m, 1, k), Dq["qweight"], Dq["scales"], Dq["qzeros"], torch.from_numpy(pos).cuda(),
                             cos, sin, heads)
        # a second call on the same workspace: the slots of the first one are zero again
        y2 = G.matmul4(g, xd, Dg["qweight"], Dg["scales"], Dg["qzeros"], Dg["bias"])
        assert torch.equal(y, y2)
        got[mode] = (y, h, r)
        assert _head_is_zero(xd.device), f"exchange mode {mode} left something in the head of the workspace"
    lib.gptq4_set_tuning(0, 0, 0)
    (yc, hc, rc), (ym, hm, rm) = got[COUNTERS], got[MARKED]
    assert torch.equal(yc, ym) and torch.equal(hc, hm)
    ref = O.quant_matmul_ref(x, gate["qweight"], gate["qzeros"], gate["scales"], g, bias=gate["bias"])
    ok, max_abs, _ = O.within_tolerance(ym.cpu().numpy(), ref)
    assert ok, max_abs
    href = O.mlp_gateup_ref(x, (gate["qweight"], gate["qzeros"], gate["scales"]), (up["qweight"], up["qzeros"], up["scales"]), g)
    assert_close(hm.cpu().numpy(), href, f"gate/up words={words} splitk={splitk} M={m}")
    if rc is not None:
        for a, b in zip(rc, rm):
            assert torch.equal(a, b)
        qr, kr, vr = O.qkv_rotary_ref(x.reshape(m, 1, k), qkv["qweight"], qkv["qzeros"], qkv["scales"], g, pos, heads, 128, max_pos=64)
        for t, want, name in zip(rm, (qr, kr, vr), "qkv"):
            assert_close(t.cpu().numpy(), want, f"{name} words={words} splitk={splitk} M={m}")


def test_default_choice_at_decode_shapes_matches_the_counter_exchange(split_k_only):
    """The automatic choice (marked values for up to 4 rows and few splits) against the forced counter exchange on
    the LLaMA-7B projections: the same bits."""
    lib = split_k_only
    G = gptq()
    for k, n in ((4096, 4096), (11008, 4096), (4096, 12288)):
        L = O.make_layer(k, n, 128, seed=k + n)
        D = to_dev(L)
        for m in (1, 3, 4, 5):
            xd = torch.from_numpy(O.make_x(m, k, seed=m)).cuda()
            lib.gptq4_set_tuning(0, 0, 0)
            y = G.matmul4(128, xd, D["qweight"], D["scales"], D["qzeros"])
            lib.gptq4_set_tuning(COUNTERS, 0, 0)
            y0 = G.matmul4(128, xd, D["qweight"], D["scales"], D["qzeros"])
            assert torch.equal(y, y0), (k, n, m)
    assert _head_is_zero(torch.device("cuda", torch.cuda.current_device()))


@pytest.mark.parametrize("kernel", ["gemv", "split_k"])
def test_a_wait_that_runs_out_sets_the_error_word_and_the_kernel_still_ends(kernel):
    """Spin limit 0xFFFFFFFF, the library's hook for this test: the finishing waves poll once and give up whatever
    they found.  The call returns, the error word of its workspace is set.  (A private workspace: it is left dirty.)"""
    from gptq_triton_amd import _lib
    lib = _lib.load()
    k, n, g, m = 4096, 4096, 128, 1
    L = O.make_layer(k, n, g, seed=5)
    D = to_dev(L)
    xd = torch.from_numpy(O.make_x(m, k, seed=6)).cuda()
    y = torch.empty((m, n), dtype=torch.float16, device="cuda")
    ws = torch.zeros(lib.gptq4_workspace_bytes(_lib.OP_MATMUL, m, k, n), dtype=torch.uint8, device="cuda")
    stream = _lib.current_stream(xd.device)

    def call():
        return lib.gptq4_matmul(xd.data_ptr(), D["qweight"].data_ptr(), D["qzeros"].data_ptr(), D["scales"].data_ptr(), None, None,
                                y.data_ptr(), m, k, n, g, ws.data_ptr(), ws.numel(), stream)

    def error_word():
        torch.cuda.synchronize()
        return int(ws[4 * _lib.WS_ERROR_WORD:4 * _lib.WS_ERROR_WORD + 4].view(torch.int32).item())

    try:
        lib.gptq4_set_gemv_tuning(2 if kernel == "gemv" else 0, 0, 0, 0)
        lib.gptq4_set_tuning(MARKED, 0, 0)
        assert call() == 0 and error_word() == 0
        ref = O.quant_matmul_ref(O.make_x(m, k, seed=6), L["qweight"], L["qzeros"], L["scales"], g)
        assert_close(y.cpu().numpy(), ref, "before the limit is lowered")
        lib.gptq4_set_exchange_spin_limit(0xFFFFFFFF)
        assert call() == 0
        assert error_word() == 1
    finally:
        lib.gptq4_set_exchange_spin_limit(0)
        lib.gptq4_set_tuning(0, 0, 0)
        lib.gptq4_set_gemv_tuning(1, 0, 0, 0)


def test_the_python_layer_reports_and_clears_an_exchange_error():
    """The module-level workspaces: after a forced give-up `check_exchange_errors` raises and names the workspace,
    `reset_workspaces` zeroes it, and the next call is right again."""
    from gptq_triton_amd import _lib
    lib = _lib.load()
    G = gptq()
    k, n, g, m = 4096, 4096, 128, 1
    L = O.make_layer(k, n, g, seed=15)
    D = to_dev(L)
    x = O.make_x(m, k, seed=16)
    xd = torch.from_numpy(x).cuda()
    _lib.check_exchange_errors()
    try:
        lib.gptq4_set_exchange_spin_limit(0xFFFFFFFF)
        G.matmul4(g, xd, D["qweight"], D["scales"], D["qzeros"])
        with pytest.raises(RuntimeError, match="gave up waiting"):
            _lib.check_exchange_errors()
    finally:
        lib.gptq4_set_exchange_spin_limit(0)
        _lib.reset_workspaces()
    assert _lib.exchange_errors() == []
    y = G.matmul4(g, xd, D["qweight"], D["scales"], D["qzeros"])
    assert_close(y.cpu().numpy(), O.quant_matmul_ref(x, L["qweight"], L["qzeros"], L["scales"], g), "after the reset")


def test_two_streams_with_a_workspace_each_do_not_disturb_each_other():
    """Calls that overlap in time on two streams (default priority), each stream with the workspace the Python layer
    keeps for it: the same bits as the same calls made alone, for the marked exchange, the counter exchange and the
    mid-M kernel's split across workgroups."""
    from gptq_triton_amd import _lib
    G = gptq()
    k, n, g = 4096, 4096, 128
    La, Lb = O.make_layer(k, n, g, seed=70), O.make_layer(11008, n, g, seed=71)
    Da, Db = to_dev(La), to_dev(Lb)
    xs = {m: torch.from_numpy(O.make_x(m, k, seed=72 + m)).cuda() for m in (1, 8, 48)}
    xb = {m: torch.from_numpy(O.make_x(m, 11008, seed=80 + m)).cuda() for m in (1, 8, 48)}
    alone_a = {m: G.matmul4(g, xs[m], Da["qweight"], Da["scales"], Da["qzeros"]) for m in xs}
    alone_b = {m: G.matmul4(g, xb[m], Db["qweight"], Db["scales"], Db["qzeros"]) for m in xb}
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    got_a, got_b = [], []
    for rep in range(40):
        for m in (1, 8, 48):
            with torch.cuda.stream(s1):
                got_a.append((m, G.matmul4(g, xs[m], Da["qweight"], Da["scales"], Da["qzeros"])))
            with torch.cuda.stream(s2):
                got_b.append((m, G.matmul4(g, xb[m], Db["qweight"], Db["scales"], Db["qzeros"])))
    torch.cuda.synchronize()
    assert all(torch.equal(y, alone_a[m]) for m, y in got_a)
    assert all(torch.equal(y, alone_b[m]) for m, y in got_b)
    _lib.check_exchange_errors()
    keys = {key[1] for key in _lib._workspaces}
    assert s1.cuda_stream in keys and s2.cuda_stream in keys
