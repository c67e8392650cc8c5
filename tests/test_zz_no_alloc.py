"""The forward entry point that allocates nothing (``vamd_lce_forward_static``) against the entry point with a
caller workspace (``vamd_lce_forward``), both through the C ABI.  The two run the same kernels, so their
outputs must be bit-equal; the second call is smaller than the first and must not see what the first left
in the built-in buffer.  Collected last on purpose: a failure here must not hide other tests from ``-x``."""
import pytest
import torch

from verl_amd import _cabi

pytestmark = pytest.mark.gpu


def _inputs(n, h, v, seed, dev):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(n, h, generator=g).bfloat16().to(dev)
    weight = (torch.randn(v, h, generator=g) * 0.05).bfloat16().to(dev)
    labels = torch.randint(0, v, (n,), generator=g).to(dev)
    return hidden, weight, labels


def _call(static, hidden, weight, labels, rcp_t, want_pi2):
    L = _cabi.lib()
    n, h = hidden.shape
    v = weight.shape[0]
    dev = hidden.device
    # poison the outputs so that an element the kernels skip cannot pass by accident
    outs = [torch.full((n,), float("nan"), device=dev, dtype=torch.float32) for _ in range(5)]
    lp, ent, lse, mz, pi2 = outs
    stream = _cabi.stream_ptr(dev)
    if static:
        rc = L.vamd_lce_forward_static(hidden.data_ptr(), weight.data_ptr(), labels.data_ptr(), n, h, v, rcp_t,
                                       lp.data_ptr(), ent.data_ptr(), lse.data_ptr(), mz.data_ptr(),
                                       pi2.data_ptr() if want_pi2 else None, stream)
    else:
        ws = _cabi.workspace(L.vamd_lce_forward_workspace_bytes(n, h, v), dev)
        rc = L.vamd_lce_forward(hidden.data_ptr(), weight.data_ptr(), labels.data_ptr(), n, h, v, rcp_t,
                                lp.data_ptr(), ent.data_ptr(), lse.data_ptr(), mz.data_ptr(), None,
                                pi2.data_ptr() if want_pi2 else None, ws.data_ptr(), ws.numel(), stream)
    _cabi.check(rc)
    torch.cuda.synchronize(dev)
    return outs if want_pi2 else outs[:4]


def test_static_forward_matches_workspace_forward_twice_second_smaller(dev):
    # first call: several token tiles and vocabulary splits, ragged in both; second: fewer tokens, narrower vocabulary
    for (n, h, v, seed, want_pi2) in ((3001, 256, 5000 // 8 * 8, 11, True), (517, 128, 1160, 12, False)):
        hidden, weight, labels = _inputs(n, h, v, seed, dev)
        want = _call(False, hidden, weight, labels, 1.0 / 1.3, want_pi2)
        got = _call(True, hidden, weight, labels, 1.0 / 1.3, want_pi2)
        for name, a, b in zip(("logprobs", "entropy", "lse", "mean_z", "sum_pi_squared"), got, want):
            assert not torch.isnan(b).any(), f"{name}: workspace entry point left elements unwritten"
            assert torch.equal(a, b), f"{name} differs at n={n}: max abs {(a - b).abs().max().item():.3e}"


def test_static_forward_refuses_more_tokens_than_its_buffer_serves(dev):
    L = _cabi.lib()
    n, h, v = 65536 + 256, 128, 256
    hidden, weight, labels = _inputs(256, h, v, 13, dev)  # never read: the size check comes first
    out = torch.empty(4, 8, device=dev)
    rc = L.vamd_lce_forward_static(hidden.data_ptr(), weight.data_ptr(), labels.data_ptr(), n, h, v, 1.0,
                                   out[0].data_ptr(), out[1].data_ptr(), out[2].data_ptr(), out[3].data_ptr(), None,
                                   _cabi.stream_ptr(dev))
    assert rc == -1
    assert b"at most 65536" in L.vamd_last_error()
