"""GPU parity of the unfused per-token definitions on materialised logits, ``clip_by_value``, the differentiable
any-axis masked reductions, the ``FusedLinearForPPO`` drop-in and the model-forward backends, against the oracle
(oracle/masked.py, oracle/head.py) evaluated on the CPU.

Tolerances: fp32 logits -> rtol 1e-5 (the kernels and the oracle both work in fp32; the ground truth is the oracle
on the same values in fp64).  bf16 / fp16 logits -> the kernels compute in fp32 and round ONCE to the input dtype,
so the result must lie within half a unit in the last place of that dtype (2**-8 resp. 2**-11 relative) of the
fp64 value, plus the fp32 slack.
"""
import math

import pytest
import torch

import oracle as O
from oracle import head as OH
from oracle import masked as OM

pytestmark = pytest.mark.gpu

HALF_ULP = {torch.float32: 0.0, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}


def _logits(n, v, dtype, seed, scale=3.0):
    g = torch.Generator().manual_seed(seed)
    z = (torch.randn(n, v, generator=g) * scale).to(dtype)
    labels = torch.randint(0, v, (n,), generator=g)
    return z, labels


def _assert_close(got, want64, dtype, what, rtol=1e-5, atol=1e-5):
    got = got.detach().double().cpu()
    err = (got - want64).abs()
    bound = atol + (rtol + HALF_ULP[dtype]) * want64.abs()
    worst = (err - bound).max().item()
    assert worst <= 0, f"{what}: max abs err {err.max().item():.3e} exceeds the bound by {worst:.3e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,v", [(1, 128), (37, 1152), (300, 1001), (5, 7), (64, 151936), (1030, 4099)])
def test_logprobs_and_entropy_from_logits_forward(dev, dtype, n, v):
    import verl_amd.utils.torch_functional as F
    z, labels = _logits(n, v, dtype, seed=n + v)
    zd, ld = z.to(dev), labels.to(dev)
    want_lp = OM.logprobs_from_logits(z.double(), labels)
    want_ent = OM.entropy_from_logits(z.double())
    for fn in (F.logprobs_from_logits, F.logprobs_from_logits_v2, F.logprobs_from_logits_naive):
        lp = fn(zd, ld)
        assert lp.shape == (n,) and lp.dtype == dtype
        _assert_close(lp, want_lp, dtype, fn.__name__)
    ent = F.entropy_from_logits(zd)
    assert ent.shape == (n,) and ent.dtype == dtype
    _assert_close(ent, want_ent, dtype, "entropy_from_logits", atol=2e-5)
    ent32 = F.entropy_from_logits_with_chunking(zd, chunk_size=64)
    assert ent32.dtype == torch.float32                              # fp32 whatever the logits are
    _assert_close(ent32, want_ent, torch.float32, "entropy_from_logits_with_chunking", atol=2e-5)
    assert (ent32 >= -1e-4).all() and (ent32 <= math.log(v) + 1e-4).all()


def test_logits_with_batch_dimensions_row_pitch_and_infinities(dev):
    import verl_amd.utils.torch_functional as F
    b, s, v = 3, 50, 777
    z, labels = _logits(b * s, v, torch.float32, seed=9)
    zd = z.view(b, s, v).to(dev)
    lp = F.logprobs_from_logits(zd, labels.view(b, s).to(dev), inplace_backward=False)
    assert lp.shape == (b, s)
    _assert_close(lp.reshape(-1), OM.logprobs_from_logits(z.double(), labels), torch.float32, "3-D logits")
    # a column slice of a wider matrix: rows are not contiguous, the kernel walks them with their pitch
    wide = torch.randn(40, 1024, generator=torch.Generator().manual_seed(1))
    lab = torch.randint(0, 900, (40,), generator=torch.Generator().manual_seed(2))
    view = wide.to(dev)[:, :900]
    assert not view.is_contiguous()
    _assert_close(F.logprobs_from_logits(view, lab.to(dev), inplace_backward=False),
                  OM.logprobs_from_logits(wide[:, :900].double(), lab), torch.float32, "strided rows")
    _assert_close(F.entropy_from_logits(view), OM.entropy_from_logits(wide[:, :900].double()), torch.float32,
                  "strided rows entropy", atol=2e-5)
    # -inf logits (a masked vocabulary): log-probs stay finite, the entropy is NaN exactly as softmax(z) * z makes it
    zi = torch.randn(4, 256, generator=torch.Generator().manual_seed(3))
    zi[:, 100:] = float("-inf")
    labi = torch.randint(0, 100, (4,), generator=torch.Generator().manual_seed(4))
    _assert_close(F.logprobs_from_logits_v2(zi.to(dev), labi.to(dev)), OM.logprobs_from_logits(zi.double(), labi),
                  torch.float32, "-inf logits")
    assert torch.isnan(OM.entropy_from_logits(zi)).all() and torch.isnan(F.entropy_from_logits(zi.to(dev))).all()
    with pytest.raises(AssertionError):
        F.logprobs_from_logits(zi.double().to(dev), labi.to(dev))                    # fp64 logits are not served
    with pytest.raises(AssertionError):
        F.logprobs_from_logits(zi.to(dev), labi[:3].to(dev))                         # label shape


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,v", [(3, 128), (130, 1152), (33, 1001), (16, 151936)])
def test_logprobs_and_entropy_from_logits_backward(dev, dtype, n, v):
    import verl_amd.utils.torch_functional as F
    z, labels = _logits(n, v, dtype, seed=3 * n + v)
    g = torch.Generator().manual_seed(n)
    g_lp, g_ent = torch.randn(n, generator=g), torch.randn(n, generator=g)
    z64 = z.double().requires_grad_()
    want_dlp, = torch.autograd.grad(OM.logprobs_from_logits(z64, labels), z64, g_lp.double())
    want_dent, = torch.autograd.grad(OM.entropy_from_logits(z64), z64, g_ent.double())
    zd = z.to(dev).requires_grad_()
    lp = F.logprobs_from_logits(zd, labels.to(dev), inplace_backward=False)
    ent = F.entropy_from_logits(zd)
    d_lp, = torch.autograd.grad(lp, zd, g_lp.to(dev).to(dtype), retain_graph=True)
    d_ent, = torch.autograd.grad(ent, zd, g_ent.to(dev).to(dtype), retain_graph=True)
    assert d_lp.dtype == dtype and d_lp.shape == (n, v)
    up_lp, up_ent = g_lp.to(dtype).double(), g_ent.to(dtype).double()          # the upstream values the kernels saw
    want_dlp = want_dlp * (up_lp / g_lp.double())[:, None]
    want_dent = want_dent * (up_ent / g_ent.double())[:, None]
    _assert_close(d_lp, want_dlp, dtype, "d logprobs / d logits", atol=1e-7)
    _assert_close(d_ent, want_dent, dtype, "d entropy / d logits", atol=1e-7)
    # both through one graph: autograd adds the two gradients
    (lp * g_lp.to(dev).to(dtype) + ent * g_ent.to(dev).to(dtype)).sum().backward()
    _assert_close(zd.grad, want_dlp + want_dent, dtype, "sum of both gradients",
                  atol=1e-7 + (1e-5 + 2 * HALF_ULP[dtype]) * (want_dlp.abs() + want_dent.abs()).max().item())


def test_inplace_backward_writes_the_gradient_over_the_logits(dev):
    import verl_amd.utils.torch_functional as F
    n, v = 20, 640
    z, labels = _logits(n, v, torch.float32, seed=5)
    z64 = z.double().requires_grad_()
    want, = torch.autograd.grad(OM.logprobs_from_logits(z64, labels).sum(), z64)
    leaf = z.to(dev).requires_grad_()
    logits = leaf * 1.0                                # a non-leaf, like model outputs divided by the temperature
    ptr = logits.data_ptr()
    lp = F.logprobs_from_logits(logits, labels.to(dev), inplace_backward=True)
    lp.sum().backward()
    _assert_close(leaf.grad, want, torch.float32, "in-place gradient", atol=1e-7)
    assert logits.data_ptr() == ptr
    _assert_close(logits, want, torch.float32, "the logits buffer now holds the gradient", atol=1e-7)


def test_clip_by_value_and_its_gradients(dev):
    import verl_amd.utils.torch_functional as F
    g = torch.Generator().manual_seed(0)
    x = torch.randn(7, 300, generator=g)
    lo = torch.randn(7, 300, generator=g) - 0.5
    hi = lo + torch.rand(7, 300, generator=g)
    x[0, :50] = hi[0, :50]            # ties with the upper bound
    x[1, :50] = lo[1, :50]            # ties with the lower bound
    hi[2, :50] = lo[2, :50]           # empty range with ties between the bounds
    up = torch.randn(7, 300, generator=g)
    cpu = [t.clone().requires_grad_() for t in (x, lo, hi)]
    want = OM.clip_by_value(*cpu)
    want_grads = torch.autograd.grad(want, cpu, up)
    gpu = [t.to(dev).requires_grad_() for t in (x, lo, hi)]
    got = F.clip_by_value(*gpu)
    assert torch.equal(got.cpu(), want.detach())
    got_grads = torch.autograd.grad(got, gpu, up.to(dev))
    for name, a, b in zip(("x", "tensor_min", "tensor_max"), got_grads, want_grads):
        assert torch.equal(a.cpu(), b), f"gradient with respect to {name}"
    # broadcast bounds: per-row minimum, scalar maximum; their gradients are summed back to their shapes
    lo_row = (lo[:, :1] - 1.0).clone().requires_grad_()
    hi_s = torch.tensor(0.3, requires_grad=True)
    xc = x.clone().requires_grad_()
    w = OM.clip_by_value(xc, lo_row, hi_s)
    wg = torch.autograd.grad(w, (xc, lo_row, hi_s), up)
    xg, lg, hg = x.to(dev).requires_grad_(), lo_row.detach().to(dev).requires_grad_(), hi_s.detach().to(dev).requires_grad_()
    o = F.clip_by_value(xg, lg, hg)
    og = torch.autograd.grad(o, (xg, lg, hg), up.to(dev))
    assert torch.equal(o.cpu(), w.detach())
    for a, b in zip(og, wg):
        assert a.shape == b.shape and torch.allclose(a.cpu(), b, rtol=1e-5, atol=1e-5)


def test_labels_outside_the_vocabulary_read_nothing(dev):
    """An ignore index (-100) or a padding id >= vocab gives a log-prob of 0 and no one-hot term in the gradient;
    the rows beside it are untouched."""
    import verl_amd.utils.torch_functional as F
    n, v = 12, 515
    z, labels = _logits(n, v, torch.float32, seed=21)
    bad = labels.clone()
    bad[3], bad[7], bad[11] = -100, v, -1
    ok = torch.ones(n, dtype=torch.bool)
    ok[[3, 7, 11]] = False
    for dtype in (torch.float32, torch.bfloat16):
        zd = z.to(dtype).to(dev).requires_grad_()
        lp = F.logprobs_from_logits(zd, bad.to(dev), inplace_backward=False)
        want = OM.logprobs_from_logits(z.to(dtype).double(), labels)
        _assert_close(lp[ok.to(dev)], want[ok], dtype, "in-range rows")
        assert (lp[~ok.to(dev)] == 0).all()
        d, = torch.autograd.grad(lp.float().sum(), zd)
        # rows without a valid label: -softmax(z), whose entries sum to -1
        row_sums = d.float().sum(-1).cpu()
        assert torch.allclose(row_sums[~ok], torch.full((3,), -1.0), atol=2e-2 if dtype != torch.float32 else 1e-5)
        assert torch.allclose(row_sums[ok], torch.zeros(int(ok.sum())), atol=2e-2 if dtype != torch.float32 else 1e-5)


def test_second_backward_through_inplace_logprobs_raises(dev):
    import verl_amd.utils.torch_functional as F
    z, labels = _logits(6, 256, torch.float32, seed=8)
    logits = z.to(dev).requires_grad_() * 1.0
    lp = F.logprobs_from_logits(logits, labels.to(dev), inplace_backward=True)
    lp.sum().backward(retain_graph=True)
    with pytest.raises(RuntimeError, match="inplace_backward"):
        lp.sum().backward()


def test_clip_by_value_hands_nan_on_like_torch(dev):
    import verl_amd.utils.torch_functional as F
    nan = float("nan")
    x = torch.tensor([nan, 0.5, 0.5, nan, 2.0, -3.0])
    lo = torch.tensor([0.0, nan, 0.0, nan, 0.0, 0.0])
    hi = torch.tensor([1.0, 1.0, nan, 1.0, 1.0, 1.0])
    up = torch.tensor([1.0, 2.0, 3.0, 4.0, 5.0, 6.0])
    cpu = [t.clone().requires_grad_() for t in (x, lo, hi)]
    want = OM.clip_by_value(*cpu)
    want_grads = torch.autograd.grad(want, cpu, up)
    gpu = [t.to(dev).requires_grad_() for t in (x, lo, hi)]
    got = F.clip_by_value(*gpu)
    assert torch.equal(torch.isnan(got.cpu()), torch.isnan(want.detach()))
    assert torch.equal(torch.nan_to_num(got.cpu(), nan=7.0), torch.nan_to_num(want.detach(), nan=7.0))
    for name, a, b in zip(("x", "tensor_min", "tensor_max"), torch.autograd.grad(got, gpu, up.to(dev)), want_grads):
        assert torch.equal(a.cpu(), b), f"gradient with respect to {name}: {a.cpu().tolist()} != {b.tolist()}"


@pytest.mark.parametrize("shift_mean", [True, False])
@pytest.mark.parametrize("mask_kind", ["bool", "weights"])
def test_masked_var_and_whiten_gradients(dev, shift_mean, mask_kind):
    """``masked_var`` / ``masked_whiten`` are plain differentiable torch in the reference
    (verl/utils/torch_functional.py:304-339); the gradients here are closed forms, compared with autograd through
    the oracle's restatement in fp64."""
    import verl_amd.utils.torch_functional as F
    g = torch.Generator().manual_seed(17)
    values = torch.randn(6, 700, generator=g) * 2.0 + 0.7
    mask = torch.rand(6, 700, generator=g) < 0.55
    mask = mask if mask_kind == "bool" else mask.float() * (0.5 + torch.rand(6, 700, generator=g))
    up = torch.randn(6, 700, generator=g)
    v64 = values.double().requires_grad_()
    m64 = mask.double() if mask_kind == "weights" else mask
    want_var = OM.masked_var(v64, m64)
    want_dvar, = torch.autograd.grad(want_var, v64)
    want_w = OM.masked_whiten(v64, m64, shift_mean)
    want_dw, = torch.autograd.grad(want_w, v64, up.double())
    vd = values.to(dev).requires_grad_()
    var = F.masked_var(vd, mask.to(dev))
    assert var.requires_grad
    assert torch.allclose(var.detach().cpu().double(), want_var.detach(), rtol=1e-5)
    dvar, = torch.autograd.grad(var, vd)
    assert torch.allclose(dvar.cpu().double(), want_dvar, rtol=1e-4, atol=1e-9), (dvar.cpu().double() - want_dvar).abs().max()
    w = F.masked_whiten(vd, mask.to(dev), shift_mean)
    assert torch.allclose(w.detach().cpu().double(), want_w.detach(), rtol=1e-5, atol=1e-5)
    dw, = torch.autograd.grad(w, vd, up.to(dev))
    err = (dw.cpu().double() - want_dw).abs().max().item()
    assert err <= 1e-5 * want_dw.abs().max().item() + 1e-7, err
    # without requires_grad nothing is recorded
    assert not F.masked_whiten(values.to(dev), mask.to(dev), shift_mean).requires_grad


@pytest.mark.parametrize("axis", [None, -1, 0, 1, 2, (0, 2), (1, 2), (0, 1, 2)])
@pytest.mark.parametrize("mask_dtype", [torch.float32, torch.bool, torch.int64])
def test_masked_sum_and_mean_any_axis_with_gradients(dev, axis, mask_dtype):
    import verl_amd.utils.torch_functional as F
    g = torch.Generator().manual_seed(4)
    values = torch.randn(4, 9, 130, generator=g)
    mask = (torch.rand(4, 9, 130, generator=g) < 0.6)
    mask[1] = False                                                    # a slab with nothing selected
    mask = mask.to(mask_dtype)
    for ref, fn in ((OM.masked_sum, F.masked_sum), (OM.masked_mean, F.masked_mean)):
        vc = values.clone().requires_grad_()
        want = ref(vc, mask, axis)
        up = torch.randn(want.shape, generator=g)
        want_grad, = torch.autograd.grad(want, vc, up)
        vd = values.to(dev).requires_grad_()
        got = fn(vd, mask.to(dev), axis)
        assert got.shape == want.shape and got.dtype == want.dtype
        assert torch.allclose(got.detach().cpu(), want.detach(), rtol=1e-5, atol=1e-5), fn.__name__
        got_grad, = torch.autograd.grad(got, vd, up.to(dev))
        assert torch.allclose(got_grad.cpu(), want_grad, rtol=1e-5, atol=1e-7), fn.__name__ + " gradient"


def test_masked_reductions_weighted_mask_nan_outside_mask_and_cpu_inputs(dev):
    import verl_amd.utils.torch_functional as F
    values = torch.tensor([[1.0, float("nan"), 3.0, 4.0], [2.0, 5.0, float("nan"), 1.0]], requires_grad=True)
    mask = torch.tensor([[1.0, 0.0, 0.5, 2.0], [1.0, 1.0, 0.0, 0.0]])
    for axis in (None, 1, 0):
        want = OM.masked_mean(values, mask, axis)
        got = F.masked_mean(values, mask, axis)                        # CPU in, CPU out
        assert got.device.type == "cpu" and torch.allclose(got, want.detach(), rtol=1e-6, equal_nan=True)
    wg, = torch.autograd.grad(OM.masked_sum(values, mask), values)
    gg, = torch.autograd.grad(F.masked_sum(values, mask), values)
    assert torch.equal(gg, wg)
    assert F.masked_sum(torch.empty(0, 3), torch.empty(0, 3)).item() == 0.0
    assert F.masked_mean(torch.empty(2, 0), torch.empty(2, 0), axis=1).tolist() == [0.0, 0.0]


@pytest.mark.parametrize("shape", [(300, 256, 2048), (2, 70, 128, 1000)])
def test_fused_linear_for_ppo_contract(dev, shape):
    """Reference contract (verl/utils/experimental/torch_functional.py:75-216): outputs in the dtype of the hidden
    states, [B, S] for 3-D input, None upstream gradients, gradients only for inputs that require them.  The
    reference's own torch-vs-torch bar (1e-4) compares two computations that share the bf16 rounding of the logits;
    this head keeps the logits in fp32, so it is held to the fp32 ground truth: the bf16 outputs must be the correctly
    rounded fp32 head outputs, within 2e-3 + half a bf16 ulp of the truth, and no further from it than the
    reference's chunked bf16 computation is."""
    from verl_amd.utils.experimental.torch_functional import FusedLinearForPPO, FusedLinearForPPOFunction
    from verl_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy
    h, v = shape[-2], shape[-1]
    lead = shape[:-2]
    n = math.prod(lead)
    g = torch.Generator().manual_seed(n + v)
    hidden = (torch.rand(n, h, generator=g) - 0.5).bfloat16()
    weight = (torch.rand(v, h, generator=g) - 0.5).bfloat16()
    ids = torch.randint(0, v, (n,), generator=g)
    T = 1.5
    want_lp, want_ent = OH.head_fp32_ground_truth(hidden, weight, ids, T)
    ref_lp, ref_ent = OH.fused_linear_for_ppo_chunked(hidden, weight, ids, T, 128)
    hd = hidden.view(*lead, h).to(dev).requires_grad_()
    wd = weight.to(dev).requires_grad_()
    idd = ids.view(*lead).to(dev).to(torch.int32)                      # the module casts ids to int64 itself
    mod = FusedLinearForPPO(chunk_size=77)
    lp, ent = mod(hd, wd, idd, temperature=T)
    assert lp.dtype == torch.bfloat16 and ent.dtype == torch.bfloat16
    assert lp.shape == tuple(lead) and ent.shape == tuple(lead)
    lp32, ent32 = linear_cross_entropy(hd.detach().view(n, h), wd.detach(), ids.to(dev), T)
    assert torch.equal(lp.reshape(-1), lp32.bfloat16()) and torch.equal(ent.reshape(-1), ent32.bfloat16())
    for got, want, ref in ((lp, want_lp, ref_lp), (ent, want_ent, ref_ent)):
        err = (got.reshape(-1).float().cpu() - want).abs()
        assert (err <= 2e-3 + 2.0 ** -8 * want.abs()).all()
        assert err.max().item() <= (ref.float() - want).abs().max().item() + 2.0 ** -8 * want.abs().max().item()
    # gradients: only d_log_probs given (d_entropy is None, not zeros), then only d_entropy
    up = torch.randn(n, generator=g).bfloat16().float()
    zero = torch.zeros(n)
    for out, (g_lp, g_ent) in ((lp, (up, zero)), (ent, (zero, up))):
        _, _, want_dh, want_dw, e_dh, e_dw = OH.head_fwd_bwd_chunked_fp32(hidden, weight, ids, T, g_lp, g_ent)
        dh, dw = torch.autograd.grad(out, (hd, wd), up.view(*lead).to(dev).bfloat16(), retain_graph=True)
        assert dh.shape == hd.shape and dh.dtype == torch.bfloat16 and dw.shape == wd.shape
        for name, a, b, e in (("d_hidden", dh.reshape(n, h), want_dh, e_dh), ("d_weight", dw, want_dw, e_dw)):
            err = (a.float().cpu() - b).abs()
            assert (err <= 2e-3 + 2.0 ** -8 * b.abs() + 2.0 ** -8 * e).all(), (name, err.max().item())
    # an input that does not require grad gets no gradient
    lp2, _ = FusedLinearForPPOFunction.apply(hd.detach(), wd, idd.to(torch.int64), T, 512)
    gw, = torch.autograd.grad(lp2.sum(), wd)
    assert gw.shape == wd.shape
    with pytest.raises(AssertionError):
        mod(hd.reshape(1, 1, n, h), wd, idd.reshape(1, 1, n))         # 4-D hidden states are refused, as there


def test_model_forward_backends_roll_labels_and_call_the_head(dev):
    from verl_amd.models.transformers import dense_common as D
    from verl_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy
    b, s, h, v = 2, 40, 128, 512
    g = torch.Generator().manual_seed(0)
    table = (torch.rand(v, h, generator=g) - 0.5).bfloat16().to(dev)
    head = (torch.rand(v, h, generator=g) - 0.5).bfloat16().to(dev)

    class Decoder(torch.nn.Module):
        def forward(self, input_ids=None, **kwargs):
            self.seen = kwargs
            return (table[input_ids],)

    class LmHead(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.weight = torch.nn.Parameter(head.clone())

    class Model(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.model, self.lm_head = Decoder(), LmHead()

        def forward(self, *args, **kwargs):
            raise AssertionError("the original forward must have been replaced")

    ids = torch.randint(0, v, (b, s), generator=g).to(dev)
    model = Model()
    D.patch_forward_with_backends(model, use_fused_kernels=False, fused_kernels_backend="hip")
    with pytest.raises(AssertionError):
        model(input_ids=ids)                                          # not patched when fused kernels are off
    D.patch_forward_with_backends(model, use_fused_kernels=True, fused_kernels_backend="triton")
    out = model(input_ids=ids, return_dict=True, temperature=1.3)
    rolled = torch.roll(ids, shifts=-1, dims=-1)
    want_lp, want_ent = linear_cross_entropy(table[ids], head, rolled, 1.3)
    assert out.log_probs.shape == (b, s) and out.log_probs.dtype == torch.float32
    assert torch.equal(out.log_probs, want_lp) and torch.equal(out.entropy, want_ent)
    out.log_probs.sum().backward()
    assert model.lm_head.weight.grad is not None
    with pytest.raises(NotImplementedError):
        model(input_ids=ids, return_dict=False)
    with pytest.raises(RuntimeError):
        D._rolled_labels(None, None, "forward_with_hip_backend")       # neither labels nor input ids
    D.patch_forward_with_backends(model, use_fused_kernels=True, fused_kernels_backend="torch")
    out_t = model(input_ids=ids, return_dict=True, temperature=1.3)
    assert out_t.log_probs.dtype == torch.bfloat16 and out_t.log_probs.shape == (b, s)
    assert torch.equal(out_t.log_probs, want_lp.bfloat16())
