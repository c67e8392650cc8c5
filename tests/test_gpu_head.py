"""GPU parity of the fused log-prob / entropy head against the oracle (fp32 stock-torch ground
truth of the reference's own test, oracle/head.py).

Tolerances (north star): max abs error 2e-3 on log-prob and entropy (fp32 outputs).  Gradients
come back in bf16 like the reference's, so on top of the 2e-3 absolute bar half a bf16 ulp of the
expected value (2**-8 relative: bf16 keeps 8 significant bits) is allowed for the final rounding of the output.  That bound is
used as is with the reference test's input distributions (|upstream grad| <= 1, |hidden| <= 0.5).
With the benchmark configs' N(0,1) hidden states and upstream gradients the d_logits entry of a
label column is O(1); like both reference implementations the kernels stage d_logits in bf16
before the two GEMMs (verl/utils/experimental/torch_functional.py:65, kernels.py:1664), which
moves each product by up to half a bf16 ulp.  Those tests add the resulting worst-case term
2**-8 * E, E = |d_logits| @ |W| resp. |d_logits|^T @ |hidden| from the oracle.
"""
import math
import random

import pytest
import torch

from oracle import head as OH
import oracle as O

pytestmark = pytest.mark.gpu

ATOL = 2e-3
BF16_HALF_ULP = 2.0 ** -8


@pytest.fixture(params=["recompute", "logits_cache"])
def backward_mode(request, monkeypatch):
    """Autograd tests run twice: with the backward pass recomputing the logits (the default) and with the opt-in
    fp32 logits cache."""
    monkeypatch.setenv("VAMD_LCE_LOGITS_CACHE_GB", "0" if request.param == "recompute" else "16")
    return request.param


def _make(n, h, v, seed, dist="uniform"):
    g = torch.Generator().manual_seed(seed)
    if dist == "uniform":          # distributions of the reference's test (uniform(-0.5, 0.5))
        hidden = torch.rand(n, h, generator=g) - 0.5
        weight = torch.rand(v, h, generator=g) - 0.5
    else:                          # distributions of the benchmark configs
        hidden = torch.randn(n, h, generator=g)
        weight = torch.randn(v, h, generator=g) * 0.02
    labels = torch.randint(0, v, (n,), generator=g)
    return hidden.bfloat16(), weight.bfloat16(), labels


def _oracle(hidden, weight, labels, T, g_lp=None, g_ent=None, device="cpu", chunk=1024):
    """fp32 ground truth, chunked over tokens so the logits stay small; grads via autograd."""
    hidden = hidden.to(device)
    weight = weight.to(device)
    labels = labels.to(device)
    want_grad = g_lp is not None or g_ent is not None
    w32 = weight.float().requires_grad_(want_grad)
    lps, ents, dhs = [], [], []
    dw = torch.zeros_like(w32) if want_grad else None
    for lo in range(0, hidden.shape[0], chunk):
        h32 = hidden[lo:lo + chunk].float().requires_grad_(want_grad)
        lp, ent = OH.head_fp32_ground_truth(h32, w32, labels[lo:lo + chunk], T)
        lps.append(lp.detach()); ents.append(ent.detach())
        if want_grad:
            outs, gos = [], []
            if g_ent is not None:
                outs.append(ent); gos.append(g_ent[lo:lo + chunk].to(device).float())
            if g_lp is not None:
                outs.append(lp); gos.append(g_lp[lo:lo + chunk].to(device).float())
            dh, dwc = torch.autograd.grad(outs, (h32, w32), gos)
            dhs.append(dh); dw += dwc
    res = [torch.cat(lps), torch.cat(ents)]
    if want_grad:
        res += [torch.cat(dhs), dw]
    return res


def _oracle_with_scale(hidden, weight, labels, T, g_lp, g_ent, device, chunk=1024):
    return OH.head_fwd_bwd_chunked_fp32(hidden.to(device), weight.to(device), labels.to(device), T,
                                        g_lp.to(device), g_ent.to(device), chunk)


def _close_bf16(got, want, what, scale=None):
    got = got.float().cpu(); want = want.float().cpu()
    err = (got - want).abs()
    bound = ATOL + BF16_HALF_ULP * want.abs()
    if scale is not None:                      # d_logits staged in bf16: half an ulp per product
        bound = bound + 2.0 ** -8 * scale.float().cpu()
    worst = (err - bound).max().item()
    assert worst <= 0, f"{what}: max abs err {err.max().item():.3e}, exceeds bound by {worst:.3e}"


@pytest.mark.parametrize("n,h,v", [(1, 128, 128), (127, 128, 384), (128, 128, 1152), (129, 256, 1152),
                                   (300, 384, 1000), (513, 128, 5000), (1388, 512, 2048)])
@pytest.mark.parametrize("T", [1.0, 1.5, 0.7])
def test_forward_small_shapes(dev, n, h, v, T):
    from verl_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy
    hidden, weight, labels = _make(n, h, v, seed=n + v)
    lp, ent = linear_cross_entropy(hidden.to(dev), weight.to(dev), labels.to(dev), T)
    want_lp, want_ent = _oracle(hidden, weight, labels, T)
    assert lp.shape == (n,) and ent.shape == (n,) and lp.dtype == torch.float32
    assert (lp.cpu() - want_lp).abs().max().item() <= ATOL
    assert (ent.cpu() - want_ent).abs().max().item() <= ATOL
    assert (lp <= 1e-6).all() and (ent >= -1e-5).all() and (ent <= math.log(v) + 1e-4).all()


@pytest.mark.parametrize("n,h,v", [(1, 128, 128), (127, 128, 384), (129, 256, 1152), (300, 384, 1000),
                                   (513, 128, 5000), (700, 256, 8192)])
@pytest.mark.parametrize("T", [1.0, 1.5])
def test_backward_small_shapes(dev, backward_mode, n, h, v, T):
    from verl_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy
    hidden, weight, labels = _make(n, h, v, seed=7 * n + v)
    g = torch.Generator().manual_seed(n)
    g_ent = (torch.rand(n, generator=g) - 0.5).bfloat16()          # bf16 upstream grads, as the reference test
    g_lp = ((torch.rand(n, generator=g) - 0.5) * 2).bfloat16()
    hd = hidden.to(dev).requires_grad_(); wd = weight.to(dev).requires_grad_()
    lp, ent = linear_cross_entropy(hd, wd, labels.to(dev), T)
    dh, dw = torch.autograd.grad((ent, lp), (hd, wd), (g_ent.to(dev).float(), g_lp.to(dev).float()))
    assert dh.dtype == torch.bfloat16 and dw.dtype == torch.bfloat16 and dh.shape == hd.shape and dw.shape == wd.shape
    _, _, want_dh, want_dw = _oracle(hidden, weight, labels, T, g_lp.float(), g_ent.float())
    _close_bf16(dh, want_dh, "d_hidden")
    _close_bf16(dw, want_dw, "d_weight")


@pytest.mark.parametrize("frozen", ["weight", "hidden"])
@pytest.mark.parametrize("n,h,v", [(129, 256, 1152), (700, 256, 8192), (1388, 512, 20000)])
def test_backward_runs_only_the_gradients_that_are_needed(dev, backward_mode, frozen, n, h, v):
    """An input that requires no gradient gets none and its GEMM is skipped (reference torch backend,
    verl/utils/experimental/torch_functional.py:150-156, :184-187); the gradient that is computed equals, bit for
    bit, the one the two-sided backward pass gives."""
    from verl_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy
    from verl_amd.utils.experimental.torch_functional import FusedLinearForPPO
    hidden, weight, labels = _make(n, h, v, seed=11 * n + v)
    g = torch.Generator().manual_seed(n + 1)
    g_ent = (torch.rand(n, generator=g) - 0.5).bfloat16().float()
    g_lp = ((torch.rand(n, generator=g) - 0.5) * 2).bfloat16().float()
    _, _, want_dh, want_dw = _oracle(hidden, weight, labels, 1.5, g_lp, g_ent)
    for op in (lambda a, b, c: linear_cross_entropy(a, b, c, 1.5), lambda a, b, c: FusedLinearForPPO()(a, b, c, 1.5)):
        hd = hidden.to(dev).requires_grad_(); wd = weight.to(dev).requires_grad_()
        lp, ent = op(hd, wd, labels.to(dev))
        both_dh, both_dw = torch.autograd.grad((ent, lp), (hd, wd), (g_ent.to(dev).to(ent.dtype), g_lp.to(dev).to(lp.dtype)))
        h1 = hidden.to(dev).requires_grad_(frozen != "hidden")
        w1 = weight.to(dev).requires_grad_(frozen != "weight")
        lp, ent = op(h1, w1, labels.to(dev))
        (ent.float() * g_ent.to(dev) + lp.float() * g_lp.to(dev)).sum().backward()
        if frozen == "weight":
            assert w1.grad is None
            _close_bf16(h1.grad, want_dh, "d_hidden with a frozen weight")
            assert torch.equal(h1.grad, both_dh)
        else:
            assert h1.grad is None
            _close_bf16(w1.grad, want_dw, "d_weight with detached hidden states")
            assert torch.equal(w1.grad, both_dw)


@pytest.mark.parametrize("n,h,v,zero_share", [(700, 256, 8192, 0.45), (1388, 512, 20000, 0.8), (300, 256, 1152, 1.0),
                                              (513, 256, 4096, 0.05)])
def test_backward_leaves_out_tokens_without_upstream_gradient(dev, monkeypatch, n, h, v, zero_share):
    """Tokens whose upstream gradients are both zero (prompt tokens under a response mask) are left out of the
    backward kernels: d_hidden is the same bits as over all tokens (zero rows where nothing came in), d_weight the
    same sum in another grouping; both against the oracle.  A share of zeros below one in ten changes nothing; a
    batch of nothing but zeros gives zero gradients without a launch."""
    from verl_amd.utils.kernel import linear_cross_entropy as K
    from verl_amd.utils.experimental.torch_functional import FusedLinearForPPO
    hidden, weight, labels = _make(n, h, v, seed=3 * n + v)
    g = torch.Generator().manual_seed(n + 7)
    g_ent = (torch.rand(n, generator=g) - 0.5).bfloat16().float()
    g_lp = ((torch.rand(n, generator=g) - 0.5) * 2).bfloat16().float()
    masked = torch.zeros(n, dtype=torch.bool)
    run = 0                                                       # runs of masked tokens, like prompts between responses
    while run < n:
        length = int(torch.randint(20, 120, (1,), generator=g))
        if torch.rand(1, generator=g).item() < zero_share:
            masked[run:run + length] = True
        run += length
    if zero_share == 1.0:
        masked[:] = True
    g_ent[masked] = 0.0
    g_lp[masked] = 0.0
    _, _, want_dh, want_dw = _oracle(hidden, weight, labels, 1.5, g_lp, g_ent)
    seen = []
    real = K.backward_over_active_tokens
    monkeypatch.setattr(K, "backward_over_active_tokens", lambda idx, *a, **k: (seen.append(int(idx.numel())), real(idx, *a, **k))[1])
    import verl_amd.utils.experimental.torch_functional as E
    monkeypatch.setattr(E, "backward_over_active_tokens", K.backward_over_active_tokens)
    for op in (lambda a, b, c: K.linear_cross_entropy(a, b, c, 1.5), lambda a, b, c: FusedLinearForPPO()(a, b, c, 1.5)):
        grads = {}
        for skip in ("1", "0"):
            monkeypatch.setenv("VAMD_LCE_SKIP_ZERO_GRAD_TOKENS", skip)
            K._ACTIVE_PROBE["rest"] = 0                           # look at the gradients in this call
            seen.clear()
            hd = hidden.to(dev).requires_grad_(); wd = weight.to(dev).requires_grad_()
            lp, ent = op(hd, wd, labels.to(dev))
            grads[skip] = torch.autograd.grad((ent, lp), (hd, wd), (g_ent.to(dev).to(ent.dtype), g_lp.to(dev).to(lp.dtype)))
            expect_compaction = skip == "1" and int(masked.sum()) * 10 >= n
            assert (seen == [n - int(masked.sum())]) if expect_compaction else (seen == []), (skip, seen)
            # a call that found (nearly) everything active is followed by calls that do not look
            assert K._ACTIVE_PROBE["rest"] == (K._ACTIVE_PROBE_REST if skip == "1" and not expect_compaction else 0)
        dh, dw = grads["1"]
        assert torch.equal(dh, grads["0"][0])
        assert (dh[masked.to(dev)] == 0).all()
        _close_bf16(dh, want_dh, "d_hidden over the active tokens")
        _close_bf16(dw, want_dw, "d_weight over the active tokens")
        _close_bf16(dw, grads["0"][1].float().cpu(), "d_weight: active tokens against all tokens")


def test_backward_c_abi_refuses_a_call_that_asks_for_nothing(dev):
    from verl_amd import _cabi
    from verl_amd.utils.kernel.linear_cross_entropy import efficient_entropy_backward, efficient_entropy_forward
    hidden, weight, labels = _make(64, 128, 256, seed=1)
    hd, wd, ld = hidden.to(dev), weight.to(dev), labels.to(dev)
    _, _, lse, mean_z = efficient_entropy_forward(hd, wd, ld)
    assert efficient_entropy_backward(None, None, hd, wd, ld, lse, mean_z, need_d_hidden=False,
                                      need_d_weight=False) == (None, None)
    L = _cabi.lib()
    ws = _cabi.workspace(L.vamd_lce_backward_workspace_bytes(64, 128, 256, 0), dev)
    rc = L.vamd_lce_backward(hd.data_ptr(), wd.data_ptr(), ld.data_ptr(), 64, 128, 256, 1.0, lse.data_ptr(),
                             mean_z.data_ptr(), None, None, 0.0, None, None, None, _cabi.DW_NONE, None, 0,
                             ws.data_ptr(), ws.numel(), _cabi.stream_ptr(dev))
    assert rc == -1 and b"neither" in L.vamd_last_error()


def _random_head_shapes(count, seed):
    rng = random.Random(seed)
    return [(rng.randint(1, 700), rng.choice([128, 256, 384, 640]), rng.randint(1, 3000), rng.choice([0.5, 1.0, 1.7]))
            for _ in range(count)]


@pytest.mark.parametrize("n,h,v,T", _random_head_shapes(14, seed=2024))
def test_random_small_shapes_fwd_bwd(dev, n, h, v, T):
    """Seeded random shapes: token counts, vocabulary sizes and hidden sizes that leave every kind of ragged tile
    (a last tile of one row or one column, vocabularies below one MFMA block, k extents of two to ten slabs)."""
    from verl_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy
    hidden, weight, labels = _make(n, h, v, seed=n * 31 + v)
    g = torch.Generator().manual_seed(v)
    g_ent = (torch.rand(n, generator=g) - 0.5).bfloat16()
    g_lp = ((torch.rand(n, generator=g) - 0.5) * 2).bfloat16()
    hd = hidden.to(dev).requires_grad_(); wd = weight.to(dev).requires_grad_()
    lp, ent = linear_cross_entropy(hd, wd, labels.to(dev), T)
    want_lp, want_ent, want_dh, want_dw, e_dh, e_dw = _oracle_with_scale(hidden, weight, labels, T, g_lp.float(),
                                                                         g_ent.float(), "cpu")
    assert (lp.cpu() - want_lp).abs().max().item() <= ATOL
    assert (ent.cpu() - want_ent).abs().max().item() <= ATOL
    dh, dw = torch.autograd.grad((ent, lp), (hd, wd), (g_ent.to(dev).float(), g_lp.to(dev).float()))
    _close_bf16(dh, want_dh, "d_hidden", e_dh)     # temperatures below 1 scale d_logits up, and with it its bf16 rounding
    _close_bf16(dw, want_dw, "d_weight", e_dw)


def test_backward_multi_chunk_and_accumulate(dev):
    """Several vocabulary chunks (fp32 d_hidden accumulation across them), entropy gradient as a
    scalar coefficient, and accumulation into an existing d_weight."""
    from verl_amd.utils.kernel import linear_cross_entropy as K
    n, h, v, T = 600, 256, 3000, 0.7
    hidden, weight, labels = _make(n, h, v, seed=11, dist="normal")
    hd, wd, ld = hidden.to(dev), weight.to(dev), labels.to(dev)
    g_lp = torch.randn(n, generator=torch.Generator().manual_seed(1))
    lp, ent, lse, mz = K.efficient_entropy_forward(hd, wd, ld, 0, T)
    dh, dw = K.efficient_entropy_backward(g_lp.to(dev), None, hd, wd, ld, lse, mz, 0, T,
                                          d_entropy_scalar=-0.001, vocab_chunk=768)
    _, _, want_dh, want_dw, e_dh, e_dw = _oracle_with_scale(hidden, weight, labels, T, g_lp, torch.full((n,), -0.001), "cpu")
    _close_bf16(dh, want_dh, "d_hidden", e_dh)
    _close_bf16(dw, want_dw, "d_weight", e_dw)
    # single-chunk path gives the same numbers up to the final rounding
    dh1, dw1 = K.efficient_entropy_backward(g_lp.to(dev), None, hd, wd, ld, lse, mz, 0, T, d_entropy_scalar=-0.001)
    _close_bf16(dh1, want_dh, "d_hidden (one chunk)", e_dh)
    _close_bf16(dw1, want_dw, "d_weight (one chunk)", e_dw)
    # cached logits instead of the recompute GEMM: same outputs, same gradients (z differs by one fp32 rounding)
    cache = torch.empty(n, v, device=dev)
    lp_c, ent_c, lse_c, mz_c = K.efficient_entropy_forward(hd, wd, ld, 0, T, logits_cache=cache)
    assert torch.equal(lp_c, lp) and torch.equal(ent_c, ent) and torch.equal(lse_c, lse) and torch.equal(mz_c, mz)
    want_z = (hidden.float() @ weight.float().t()) / T
    assert (cache.cpu() - want_z).abs().max().item() <= 1e-4 * want_z.abs().max().item() + 1e-5
    for chunk in (768, 0):
        dh_c, dw_c = K.efficient_entropy_backward(g_lp.to(dev), None, hd, wd, ld, lse, mz, 0, T,
                                                  d_entropy_scalar=-0.001, vocab_chunk=chunk, logits_cache=cache)
        _close_bf16(dh_c, want_dh, "d_hidden (cached logits)", e_dh)
        _close_bf16(dw_c, want_dw, "d_weight (cached logits)", e_dw)
    # accumulate: second call adds into the first call's d_weight
    dw_acc = dw1.clone()
    K.efficient_entropy_backward(g_lp.to(dev), None, hd, wd, ld, lse, mz, 0, T, d_entropy_scalar=-0.001,
                                 d_weight_out=dw_acc)
    _close_bf16(dw_acc, 2 * want_dw, "d_weight accumulated twice", 2 * e_dw + 2.0 * want_dw.abs())


def test_reductions_3d_input_and_argument_errors(dev):
    from verl_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy
    b, s, h, v = 2, 70, 128, 512
    hidden, weight, labels = _make(b * s, h, v, seed=3)
    hd = hidden.view(b, s, h).to(dev).requires_grad_()
    wd = weight.to(dev).requires_grad_()
    ld = labels.view(b, s).to(dev)
    lp, ent = linear_cross_entropy(hd, wd, ld, 1.5, "none")
    assert lp.shape == (b, s) and ent.shape == (b, s)                        # batch-shaped for batched input
    want_lp, want_ent, want_dh, want_dw = _oracle(hidden, weight, labels, 1.5, torch.ones(b * s), torch.zeros(b * s))
    assert (lp.reshape(-1) - want_lp.to(dev)).abs().max().item() <= ATOL
    assert (lp[:, -5:-1].reshape(-1) - want_lp.view(b, s)[:, -5:-1].reshape(-1).to(dev)).abs().max().item() <= ATOL
    up = torch.randn(b, s, generator=torch.Generator().manual_seed(1)).to(dev)
    dh_b, = torch.autograd.grad((lp * up).sum(), hd)                         # batch-shaped upstream gradients
    lp_flat, _ = linear_cross_entropy(hd.view(b * s, h), wd, ld.view(-1), 1.5, "none")
    assert lp_flat.shape == (b * s,)                                         # flat for 2-D input, like the reference op
    dh_f, = torch.autograd.grad((lp_flat * up.view(-1)).sum(), hd)
    assert torch.equal(dh_b, dh_f)
    lp_sum, _ = linear_cross_entropy(hd, wd, ld, 1.5, "sum")
    lp_mean, _ = linear_cross_entropy(hd, wd, ld, 1.5, "MEAN")
    assert lp_sum.dim() == 0 and abs(lp_sum.item() - want_lp.sum().item()) <= ATOL * b * s
    assert abs(lp_mean.item() - want_lp.mean().item()) <= ATOL
    dh, dw = torch.autograd.grad(lp_sum, (hd, wd))
    assert dh.shape == hd.shape
    _close_bf16(dh.view(b * s, h), want_dh, "d_hidden (sum)")
    _close_bf16(dw, want_dw, "d_weight (sum)")
    with pytest.raises(ValueError):
        linear_cross_entropy(hd, wd, ld, 1.5, "max")
    with pytest.raises(AssertionError):
        linear_cross_entropy(hd, wd, ld, 1, "none")                          # temperature must be a float
    with pytest.raises(AssertionError):
        linear_cross_entropy(hd.float(), wd.float(), ld, 1.5, "none")        # bf16 only
    with pytest.raises(AssertionError):
        linear_cross_entropy(hd[..., :64], wd[:, :64], ld, 1.5, "none")      # non-contiguous / H % 128


@pytest.mark.parametrize("case", [0, 1, 2, 3, 4])
def test_reference_test_shapes_fwd_bwd(dev, backward_mode, case):
    """The five (N, H, V) cases of the reference's own test (tests/utils/test_linear_cross_entropy.py:112-143),
    its input distributions and bf16 upstream grads; ground truth evaluated in fp32 on the GPU."""
    from conftest import load_golden
    fx = load_golden()["head_shapes"]
    n, h, v = (fx["cases"][case][k] for k in ("num_tokens", "hidden_size", "vocab"))
    T = fx["temperature"]
    from verl_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy
    hidden, weight, labels = _make(n, h, v, seed=5)
    g = torch.Generator().manual_seed(6)
    g_ent = (torch.rand(n, generator=g) - 0.5).bfloat16().float()
    g_lp = ((torch.rand(n, generator=g) - 0.5) * 2).bfloat16().float()
    hd = hidden.to(dev).requires_grad_(); wd = weight.to(dev).requires_grad_()
    lp, ent = linear_cross_entropy(hd, wd, labels.to(dev), T)
    dh, dw = torch.autograd.grad((ent, lp), (hd, wd), (g_ent.to(dev), g_lp.to(dev)))
    want_lp, want_ent, want_dh, want_dw = _oracle(hidden, weight, labels, T, g_lp, g_ent, device=dev, chunk=512)
    assert (lp - want_lp).abs().max().item() <= ATOL
    assert (ent - want_ent).abs().max().item() <= ATOL
    _close_bf16(dh, want_dh, "d_hidden")
    _close_bf16(dw, want_dw, "d_weight")


def test_benchmark_config_7b_head_full_size(dev):
    """Full Qwen2.5-7B head shape (N=16384, H=3584, V=152064, T=1, dlogprob ~ N(0,1), dentropy =
    0.001): every output compared with the fp32 ground truth evaluated on the GPU in 1024-token
    chunks, plus size-independent properties (entropy in [0, log V], log-prob <= 0, softmax
    gradient rows summing to zero over the vocabulary, linearity in the upstream gradient)."""
    from verl_amd.utils.kernel import linear_cross_entropy as K
    n, h, v, T = 16384, 3584, 152064, 1.0
    g = torch.Generator(device=dev).manual_seed(0)
    hidden = torch.randn(n, h, device=dev, generator=g).bfloat16()
    weight = (torch.randn(v, h, device=dev, generator=g) * 0.02).bfloat16()
    labels = torch.randint(0, v, (n,), device=dev, generator=g)
    g_lp = torch.randn(n, device=dev, generator=g)
    g_ent = torch.full((n,), 0.001, device=dev)
    lp, ent, lse, mz = K.efficient_entropy_forward(hidden, weight, labels, 0, T)
    dh, dw = K.efficient_entropy_backward(g_lp, None, hidden, weight, labels, lse, mz, 0, T, d_entropy_scalar=0.001)
    assert (lp <= 0).all() and (ent >= 0).all() and (ent <= math.log(v) + 1e-4).all()
    want_lp, want_ent, want_dh, want_dw, e_dh, e_dw = _oracle_with_scale(hidden, weight, labels, T, g_lp, g_ent, dev)
    assert (lp - want_lp).abs().max().item() <= ATOL
    assert (ent - want_ent).abs().max().item() <= ATOL
    _close_bf16(dh, want_dh, "d_hidden", e_dh)
    _close_bf16(dw, want_dw, "d_weight", e_dw)
    # measured errors against the strict 2e-3 (printed with -s; the gradients' share beyond 2e-3 is the bf16
    # rounding of the outputs and of the staged d_logits, which the bound above spells out)
    errs = {"logprob": (lp - want_lp).abs().max().item(), "entropy": (ent - want_ent).abs().max().item(),
            "d_hidden": (dh.float() - want_dh).abs().max().item(), "d_weight": (dw.float() - want_dw).abs().max().item()}
    rms = {"d_hidden": (dh.float() - want_dh).pow(2).mean().sqrt().item(),
           "d_weight": (dw.float() - want_dw).pow(2).mean().sqrt().item()}
    frac_over = {"d_hidden": ((dh.float() - want_dh).abs() > ATOL).float().mean().item(),
                 "d_weight": ((dw.float() - want_dw).abs() > ATOL).float().mean().item()}
    print(f"\nC2 recompute: max abs err {errs}; rms {rms}; share of elements beyond 2e-3 {frac_over}; "
          f"max |d_hidden| {want_dh.abs().max().item():.3e}, max |d_weight| {want_dw.abs().max().item():.3e}")
    # typical (not worst-case) agreement: the rms error stays below half a bf16 ulp (2**-8) of the rms gradient,
    # i.e. on average the result is as close as its own output format allows
    rel = {"d_hidden": rms["d_hidden"] / want_dh.pow(2).mean().sqrt().item(),
           "d_weight": rms["d_weight"] / want_dw.pow(2).mean().sqrt().item()}
    print(f"C2 recompute: rms error / rms gradient {rel}")
    assert rel["d_hidden"] < BF16_HALF_ULP and rel["d_weight"] < BF16_HALF_ULP, rel
    assert errs["logprob"] < 1e-4 and errs["entropy"] < 1e-4 and errs["d_hidden"] < ATOL, errs
    del want_dw, want_dh, e_dw, e_dh
    # sum_j dz_j = 0 for every token  =>  the vocabulary-axis sum of d_weight vanishes (bf16 rounding of 152064 rows)
    # (each of the ~16384 label rows carries its own bf16 rounding error, so the sum is noise of relative size ~1e-5)
    col_sum = dw.float().sum(0)
    col_abs = dw.float().abs().sum(0)
    assert (col_sum.abs() <= 1e-3 * col_abs).all(), (col_sum.abs() / col_abs).max().item()
    # linearity in the upstream gradient: backward(2 g) == 2 backward(g) up to output rounding
    dh2, _ = K.efficient_entropy_backward(2 * g_lp, None, hidden, weight, labels, lse, mz, 0, T, d_entropy_scalar=0.002)
    _close_bf16(dh2, 2 * dh.float(), "linearity of d_hidden")
    del dh2
    # cached-logits path at full size: identical forward outputs; gradients differ from the recompute path only
    # where one fp32 rounding of z moves a d_logits entry across a bf16 rounding boundary
    cache = torch.empty(n, v, device=dev)
    lp_c, ent_c, lse_c, mz_c = K.efficient_entropy_forward(hidden, weight, labels, 0, T, logits_cache=cache)
    assert torch.equal(lp_c, lp) and torch.equal(ent_c, ent)
    dh_c, dw_c = K.efficient_entropy_backward(g_lp, None, hidden, weight, labels, lse_c, mz_c, 0, T,
                                              d_entropy_scalar=0.001, logits_cache=cache)
    del cache
    print(f"C2 logits cache vs recompute: max abs diff d_hidden {(dh_c.float() - dh.float()).abs().max().item():.3e}, "
          f"d_weight {(dw_c.float() - dw.float()).abs().max().item():.3e}")
    _close_bf16(dh_c, dh.float(), "d_hidden cached vs recomputed")
    _close_bf16(dw_c, dw.float(), "d_weight cached vs recomputed")
    assert (dh_c.float() - dh.float()).pow(2).mean().sqrt().item() < 1e-4
    assert (dw_c.float() - dw.float()).pow(2).mean().sqrt().item() < 1e-4


def test_benchmark_config_small_head_forward_only(dev):
    """Qwen2.5-0.5B head shape, forward only (N=2048, H=896, V=151936, T=1): the configuration the reference's CPU
    path runs in full."""
    from verl_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy
    n, h, v, T = 2048, 896, 151936, 1.0
    hidden, weight, labels = _make(n, h, v, seed=21, dist="normal")
    with torch.no_grad():
        lp, ent = linear_cross_entropy(hidden.to(dev), weight.to(dev), labels.to(dev), T)
    want_lp, want_ent = _oracle(hidden, weight, labels, T, device=dev)
    assert lp.dtype == torch.float32 and lp.shape == (n,)
    assert (lp - want_lp).abs().max().item() <= ATOL and (ent - want_ent).abs().max().item() <= ATOL


def test_benchmark_config_llama_head_token_chunked(dev):
    """Llama-3.1-8B head shape at long-rollout scale (N=65536, H=4096, V=128256, T=0.7) processed in eight
    8192-token chunks, the entropy coefficient 0.001 passed as a scalar folded into the backward.  The weight
    gradient is summed over the eight chunks in fp32 and rounded to bf16 once, so it is held to the same bound as
    a single call.  Alternating chunks go through the logits cache and through the recompute path.  The same sum
    kept in bf16 (one rounding of the running sum per chunk, what ``weight.grad +=`` does in bf16 training) is run
    beside it and must stay within one extra half-ulp of the running value per accumulation."""
    from verl_amd.utils.kernel import linear_cross_entropy as K
    n, h, v, T, chunk = 65536, 4096, 128256, 0.7, 8192
    g = torch.Generator(device=dev).manual_seed(5)
    hidden = torch.randn(n, h, device=dev, generator=g).bfloat16()
    weight = (torch.randn(v, h, device=dev, generator=g) * 0.02).bfloat16()
    labels = torch.randint(0, v, (n,), device=dev, generator=g)
    g_lp = torch.randn(n, device=dev, generator=g)
    acc32 = torch.empty(v, h, device=dev, dtype=torch.float32)
    d_weight_bf16_sum = torch.zeros_like(weight)
    lps, ents, dhs = [], [], []
    d_weight = None
    n_chunks = n // chunk
    for ci, lo in enumerate(range(0, n, chunk)):
        sl = slice(lo, lo + chunk)
        cache = torch.empty(chunk, v, device=dev) if ci % 2 == 0 else None
        lp, ent, lse, mz = K.efficient_entropy_forward(hidden[sl], weight, labels[sl], 0, T, logits_cache=cache)
        step = "first" if ci == 0 else ("last" if ci == n_chunks - 1 else "middle")
        dh, dw = K.efficient_entropy_backward(g_lp[sl], None, hidden[sl], weight, labels[sl], lse, mz, 0, T,
                                              d_entropy_scalar=0.001, logits_cache=cache,
                                              d_weight_acc32=acc32, acc32_step=step)
        assert (dw is None) == (step != "last")
        d_weight = dw
        dh2, _ = K.efficient_entropy_backward(g_lp[sl], None, hidden[sl], weight, labels[sl], lse, mz, 0, T,
                                              d_entropy_scalar=0.001, logits_cache=cache,
                                              d_weight_out=d_weight_bf16_sum)
        assert torch.equal(dh, dh2)
        lps.append(lp); ents.append(ent); dhs.append(dh)
        del cache
    del acc32
    want_lp, want_ent, want_dh, want_dw, e_dh, e_dw = _oracle_with_scale(
        hidden, weight, labels, T, g_lp, torch.full((n,), 0.001, device=dev), dev)
    assert (torch.cat(lps) - want_lp).abs().max().item() <= ATOL
    assert (torch.cat(ents) - want_ent).abs().max().item() <= ATOL
    _close_bf16(torch.cat(dhs), want_dh, "d_hidden", e_dh)
    _close_bf16(d_weight, want_dw, "d_weight summed over 8 token chunks in fp32", e_dw)
    # the bf16 running sum: each of the 7 additions rounds a value no larger than the final one in magnitude plus
    # what is still to come; bound it by half an ulp of (|want| + E) per accumulation
    _close_bf16(d_weight_bf16_sum, want_dw, "d_weight summed over 8 token chunks in bf16",
                e_dw + (n_chunks - 1) * (want_dw.abs() + e_dw))
    err32 = (d_weight.float() - want_dw).abs().max().item()
    err16 = (d_weight_bf16_sum.float() - want_dw).abs().max().item()
    print(f"\nC5 d_weight max abs err: fp32 accumulation {err32:.3e}, bf16 accumulation {err16:.3e}; "
          f"max |d_weight| {want_dw.abs().max().item():.3e}")


def test_weight_gradient_fp32_accumulation_small(dev):
    """Three token chunks summed in fp32 equal one call over all tokens up to the final bf16 rounding."""
    from verl_amd.utils.kernel import linear_cross_entropy as K
    n, h, v, T = 900, 256, 3000, 1.3
    hidden, weight, labels = _make(n, h, v, seed=17, dist="normal")
    hd, wd, ld = hidden.to(dev), weight.to(dev), labels.to(dev)
    g_lp = torch.randn(n, generator=torch.Generator().manual_seed(2)).to(dev)
    g_ent = torch.full((n,), 0.01, device=dev)
    acc32 = torch.full((v, h), float("nan"), device=dev)        # "first" must overwrite, not add
    out = torch.empty_like(wd)
    for step, sl in (("first", slice(0, 300)), ("middle", slice(300, 650)), ("last", slice(650, 900))):
        _, _, lse, mz = K.efficient_entropy_forward(hd[sl], wd, ld[sl], 0, T)
        _, dw = K.efficient_entropy_backward(g_lp[sl], g_ent[sl], hd[sl], wd, ld[sl], lse, mz, 0, T,
                                             d_weight_acc32=acc32, acc32_step=step, d_weight_out=out, vocab_chunk=1024)
    assert dw is out
    _, _, want_dh, want_dw, e_dh, e_dw = _oracle_with_scale(hidden, weight, labels, T, g_lp.cpu(), g_ent.cpu(), "cpu")
    _close_bf16(out, want_dw, "d_weight (fp32 accumulation, 3 chunks)", e_dw)
    assert torch.equal(out, acc32.bfloat16())


@pytest.mark.parametrize("n,h,v", [(130, 128, 1001), (257, 256, 257), (64, 128, 7), (300, 128, 4099)])
def test_vocabulary_not_a_multiple_of_eight(dev, n, h, v):
    """The vocabulary tail is masked, as in the reference (kernels.py masks ragged V); forward and backward."""
    from verl_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy
    hidden, weight, labels = _make(n, h, v, seed=n + v)
    g = torch.Generator().manual_seed(v)
    g_lp, g_ent = torch.randn(n, generator=g), torch.randn(n, generator=g) * 0.1
    hd = hidden.to(dev).requires_grad_(); wd = weight.to(dev).requires_grad_()
    lp, ent = linear_cross_entropy(hd, wd, labels.to(dev), 1.2)
    dh, dw = torch.autograd.grad((lp, ent), (hd, wd), (g_lp.to(dev), g_ent.to(dev)))
    want_lp, want_ent, want_dh, want_dw, e_dh, e_dw = _oracle_with_scale(hidden, weight, labels, 1.2, g_lp, g_ent, "cpu")
    assert (lp.cpu() - want_lp).abs().max().item() <= ATOL and (ent.cpu() - want_ent).abs().max().item() <= ATOL
    _close_bf16(dh, want_dh, "d_hidden", e_dh)
    _close_bf16(dw, want_dw, "d_weight", e_dw)


def test_head_forward_backward_replays_from_a_hip_graph(dev):
    """The head's entry points allocate nothing and clear nothing with memset, so a forward + backward (recompute
    mode, three vocabulary chunks) can be captured once and replayed: three replays on fresh operands, eager work
    in between, each bit-equal to the eager calls."""
    from verl_amd import _cabi
    Lb = _cabi.lib()
    n, h, v, T = 600, 256, 3000, 0.7
    gen = torch.Generator(device=dev).manual_seed(9)
    hidden = torch.empty(n, h, device=dev, dtype=torch.bfloat16)
    weight = torch.empty(v, h, device=dev, dtype=torch.bfloat16)
    labels = torch.empty(n, device=dev, dtype=torch.int64)
    g_lp = torch.empty(n, device=dev)
    chunk = 1024
    ws_f = torch.empty(Lb.vamd_lce_forward_workspace_bytes(n, h, v), dtype=torch.uint8, device=dev)
    ws_b = torch.empty(Lb.vamd_lce_backward_workspace_bytes(n, h, v, chunk), dtype=torch.uint8, device=dev)

    def outputs():
        f = lambda: torch.empty(n, device=dev)
        return dict(lp=f(), ent=f(), lse=f(), mz=f(), dh=torch.empty_like(hidden), dw=torch.empty_like(weight))

    def step(o):
        st = _cabi.stream_ptr(dev)
        P = lambda t: t.data_ptr()
        _cabi.check(Lb.vamd_lce_forward(P(hidden), P(weight), P(labels), n, h, v, 1.0 / T, P(o["lp"]), P(o["ent"]),
                                        P(o["lse"]), P(o["mz"]), None, None, P(ws_f), ws_f.numel(), st))
        _cabi.check(Lb.vamd_lce_backward(P(hidden), P(weight), P(labels), n, h, v, 1.0 / T, P(o["lse"]), P(o["mz"]),
                                         P(g_lp), None, 0.001, None, P(o["dh"]), P(o["dw"]), _cabi.DW_STORE, None,
                                         chunk, P(ws_b), ws_b.numel(), st))

    def refill():
        hidden.copy_(torch.randn(n, h, device=dev, generator=gen).bfloat16())
        weight.copy_((torch.randn(v, h, device=dev, generator=gen) * 0.05).bfloat16())
        labels.copy_(torch.randint(0, v, (n,), device=dev, generator=gen))
        g_lp.copy_(torch.randn(n, device=dev, generator=gen))

    refill()
    captured = outputs()
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        step(captured)                                           # warm-up outside the capture
    torch.cuda.current_stream(dev).wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(captured)
    for _ in range(3):
        refill()
        eager = outputs()
        step(eager)
        torch.cuda.synchronize()
        for t in captured.values():
            t.fill_(float("nan")) if t.is_floating_point() else None
        graph.replay()
        torch.cuda.synchronize()
        for name in eager:
            assert torch.equal(captured[name], eager[name]), name
    want = OH.head_fp32_ground_truth(hidden.cpu(), weight.cpu(), labels.cpu(), T)
    assert (captured["lp"].cpu() - want[0]).abs().max().item() <= ATOL


@pytest.mark.parametrize("shape", [0, 1])
def test_mfma_yardstick_runs_and_counts_its_flops(dev, shape):
    """The register-only matrix-instruction loop of the benchmark: with every operand 1.0 each accumulator grows by
    the instruction's k extent per round, so the sum a thread reports is known exactly."""
    from verl_amd import _cabi
    Lb = _cabi.lib()
    wgs, iters = 4, 3
    ones = torch.full((wgs * 512 * 32,), 0x3F803F80, dtype=torch.int32, device=dev)      # two bf16 1.0 per word
    out = torch.empty(wgs * 512, device=dev)
    _cabi.check(Lb.vamd_mfma_yardstick(shape, ones.data_ptr(), out.data_ptr(), wgs, iters, _cabi.stream_ptr(dev)))
    torch.cuda.synchronize()
    k, accs = (16, 8 * 16) if shape == 0 else (32, 32 * 4)      # k per instruction; accumulator values per thread
    assert torch.equal(out, torch.full_like(out, float(iters * k * accs)))
    per_wave = (8 * 32768) if shape == 0 else (32 * 16384)
    assert Lb.vamd_mfma_yardstick_flops(shape, wgs, iters) == wgs * 8 * iters * per_wave
    assert Lb.vamd_mfma_yardstick(7, ones.data_ptr(), out.data_ptr(), wgs, iters, _cabi.stream_ptr(dev)) != 0


def test_forward_without_grad_keeps_no_logits(dev, monkeypatch):
    """Under torch.no_grad() (the actor's compute_log_prob) no [tokens, vocab] tensor is allocated even when the
    weight requires grad and the logits cache is switched on."""
    from verl_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy
    monkeypatch.setenv("VAMD_LCE_LOGITS_CACHE_GB", "16")
    n, h, v = 4096, 256, 32768
    hidden, weight, labels = _make(n, h, v, seed=1)
    hd, wd, ld = hidden.to(dev), weight.to(dev).requires_grad_(), labels.to(dev)
    torch.cuda.synchronize(); torch.cuda.reset_peak_memory_stats(dev)
    base = torch.cuda.memory_allocated(dev)
    with torch.no_grad():
        lp, ent = linear_cross_entropy(hd, wd, ld, 1.0)
    torch.cuda.synchronize()
    assert torch.cuda.max_memory_allocated(dev) - base < 4 * n * v // 8
    assert not lp.requires_grad
    # with grad mode on and the cache switched on, the same call does keep the logits
    torch.cuda.reset_peak_memory_stats(dev)
    lp2, _ = linear_cross_entropy(hd, wd, ld, 1.0)
    assert torch.cuda.max_memory_allocated(dev) - base >= 4 * n * v and torch.equal(lp2.detach(), lp)
    # and by default (cache off) it does not
    monkeypatch.setenv("VAMD_LCE_LOGITS_CACHE_GB", "0")
    del lp2
    torch.cuda.synchronize(); torch.cuda.reset_peak_memory_stats(dev)
    base = torch.cuda.memory_allocated(dev)
    lp3, _ = linear_cross_entropy(hd, wd, ld, 1.0)
    assert torch.cuda.max_memory_allocated(dev) - base < 4 * n * v // 8 and lp3.requires_grad


@pytest.mark.parametrize("n,h,v,T", [(1, 128, 128, 1.0), (300, 384, 1000, 0.7), (700, 256, 8192, 1.5), (2169, 896, 151936, 1.0)])
def test_sum_pi_squared_from_the_head(dev, n, h, v, T):
    """sum_j softmax(z)_j^2 carried by the forward pass next to log-prob and entropy; the other outputs are the
    same numbers the plain forward gives."""
    from verl_amd.utils.kernel import linear_cross_entropy as K
    from oracle import masked as OM
    hidden, weight, labels = _make(n, h, v, seed=3 * n + v, dist="normal" if v > 10000 else "uniform")
    hd, wd, ld = hidden.to(dev), weight.to(dev), labels.to(dev)
    lp, ent, pi2 = K.linear_cross_entropy_with_sum_pi_squared(hd, wd, ld, T)
    lp0, ent0, _, _ = K.efficient_entropy_forward(hd, wd, ld, 0, T)
    assert torch.equal(lp, lp0) and torch.equal(ent, ent0)
    want = []
    for lo in range(0, n, 512):
        z = (hd[lo:lo + 512].float() @ wd.float().t()) / T
        want.append(OM.sum_pi_squared_from_logits(z))
    want = torch.cat(want)
    assert pi2.shape == (n,) and pi2.dtype == torch.float32
    assert (pi2 >= 1.0 / v - 1e-9).all() and (pi2 <= 1.0 + 1e-6).all()
    assert torch.allclose(pi2, want, rtol=2e-3, atol=1e-9), ((pi2 - want).abs() / want).max().item()


@pytest.mark.parametrize("geometry", [(2, 5, 2), (8, 96, 64), (16, 1500, 1499), (4, 64, 1)])
def test_pad_to_response_window(dev, geometry):
    """The remove-padding outputs land in the response window exactly as pad_input + slice place them, and the
    upstream gradients come back to the tokens (reference dp_actor.py:316-344)."""
    from verl_amd.utils.kernel.response_window import pad_to_response_window
    B, S, Lr = geometry
    g = torch.Generator().manual_seed(B * S + Lr)
    left = torch.randint(0, S // 2 + 1, (B,), generator=g)       # left padding of the prompt
    right = torch.randint(0, S // 2, (B,), generator=g)          # right padding of the response
    pos = torch.arange(S)[None, :]
    attention = ((pos >= left[:, None]) & (pos < (S - right)[:, None])).long()
    attention[0] = 1
    indices = attention.flatten().nonzero().flatten()
    nnz = indices.numel()
    vals = [torch.randn(nnz, generator=g) for _ in range(3)]
    dv = [v.to(dev).requires_grad_() for v in vals[:2]] + [vals[2].to(dev)]
    got = pad_to_response_window(indices.to(dev), B, S, Lr, *dv)
    assert len(got) == 3
    ov = [v.clone().requires_grad_() for v in vals]
    want = [O.pad_to_response_window(v, indices, B, S, Lr) for v in ov]
    for a, b in zip(got, want):
        assert a.shape == (B, Lr) and torch.equal(a.cpu(), b.detach())
    up = [torch.randn(B, Lr, generator=g) for _ in range(2)]
    (got[0] * up[0].to(dev)).sum().add((got[1] * up[1].to(dev)).sum()).backward()
    (want[0] * up[0]).sum().add((want[1] * up[1]).sum()).backward()
    assert torch.equal(dv[0].grad.cpu(), ov[0].grad) and torch.equal(dv[1].grad.cpu(), ov[1].grad)
    only, = pad_to_response_window(indices.to(dev), B, S, Lr, vals[0].to(dev))
    assert torch.equal(only.cpu(), want[0].detach())
