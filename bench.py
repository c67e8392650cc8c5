"""Benchmark of the hot path on one MI355X: fused log-prob + entropy head, forward + backward,
at the Qwen2.5-7B head shape (hidden [16384, 3584] bf16, weight [152064, 3584] bf16, T = 1,
dlogprob ~ N(0,1) fp32, dentropy = 0.001).

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  ``value`` is tokens/s of forward+backward with inputs resident in HBM.
``roofline`` describes the kernel that takes the most time in a step, from HIP events recorded
around every launch on the launch stream; ``cpu_baseline`` times the CPU oracle (the reference's
chunked PyTorch backend restated) on a bounded token sample of the same workload.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
KERNEL_NAMES = ["lce_forward_kernel", "lce_merge_kernel", "lce_recompute_kernel", "lce_dgrad_kernel", "lce_dlogits_kernel"]
# MFMA GEMMs of 2*N*V*H flops each that a kernel performs per step
COPY_YARDSTICK_BYTES = 1 << 30
# L2 <-> fabric bytes of one full-chunk launch (16384 vocabulary columns) of each kernel at this workload come from
# counter passes (rocprofv3 FETCH_SIZE and WRITE_SIZE, scaled by the readings of the 1 GiB copy in the same run).
# Counters cannot be read from inside this process, so the pass that writes profiles/head_fwd_bwd_qwen7b_hbm_traffic.md
# also writes the figures, with the commit they were taken at, to this file; the bench line quotes both.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "head_traffic.json")


def measured_traffic(kernel: str):
    """(bytes per full-chunk launch, commit of the measurement) of `kernel`, or (None, None) without a counter pass."""
    try:
        rec = json.load(open(TRAFFIC_FILE))
        fetch, write = rec["bytes_per_launch"][kernel]
        return float(fetch) + float(write), rec.get("commit")
    except (OSError, KeyError, ValueError, TypeError):
        return None, None


GEMMS_PER_STEP = {"lce_forward_kernel": 1, "lce_recompute_kernel": 1, "lce_dgrad_kernel": 2}


def cpu_baseline(n_cpu: int, h: int, v: int, temperature: float) -> dict:
    """The reference's chunked torch backend (oracle port) on `n_cpu` tokens of the same workload."""
    import torch

    import oracle as O

    torch.set_num_threads(os.cpu_count() or 1)
    g = torch.Generator().manual_seed(1)
    hidden = torch.randn(n_cpu, h, generator=g).bfloat16()
    weight = (torch.randn(v, h, generator=g) * 0.02).bfloat16()
    labels = torch.randint(0, v, (n_cpu,), generator=g)
    g_lp = torch.randn(n_cpu, generator=g)
    g_ent = torch.full((n_cpu,), 0.001)
    t0 = time.perf_counter()
    O.fused_linear_for_ppo_chunked(hidden, weight, labels, temperature, 512, g_lp, g_ent)
    dt = time.perf_counter() - t0
    return {
        "value": n_cpu / dt,
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{n_cpu} of 16384 tokens (full vocab and hidden size), chunked torch backend, bf16 GEMMs, "
                  f"fwd+bwd once, {dt:.1f} s; tokens/s scales linearly in tokens",
    }


def policy_math_rates(dev, with_cpu: bool, B: int = 512, Lc: int = 4096, n_groups: int = 64, only=None,
                      buffer_sets: int | None = None) -> dict:
    """The [B, L] kernels (B = 512, L = 4096 is the size of the GRPO / policy-loss and GAE benchmark configurations): microseconds per call from HIP events
    over 48 calls (best of three such loops) that rotate through 8 buffer sets, 16 at the smaller size (so that even the two-tensor ops
    touch more than the 256 MB Infinity Cache before they come back to a set), the algorithmic bytes of
    the op, and the fraction of 8 TB/s that gives.  ``cpu_ms`` is the CPU oracle on one buffer set.
    ``buffer_sets=1`` times the same calls on one set that stays in the caches (what a kernel sees whose inputs the
    kernel before it has just written): how much of a call at this size is waiting for memory at all."""
    import torch

    import oracle as O
    from verl_amd import _cabi

    L = _cabi.lib()
    BL = B * Lc
    nset = 16 if BL * 4 * 2 * 8 < (300 << 20) else 8   # two fp32 tensors per set must add up to more than the cache
    if buffer_sets is not None:
        nset = buffer_sets
    g = torch.Generator(device=dev).manual_seed(0)

    def mk():
        lens = torch.randint(64, Lc + 1, (B,), device=dev, generator=g)
        mask = (torch.arange(Lc, device=dev)[None, :] < lens[:, None]).float()
        t = lambda: torch.randn(B, Lc, device=dev, generator=g)
        return dict(mask=mask, a=t(), b=t(), c=t(), o1=torch.empty(B, Lc, device=dev),
                    o2=torch.empty(B, Lc, device=dev))

    sets = [mk() for _ in range(nset)]
    ws_bytes = max(1 << 22, L.vamd_policy_loss_variant_workspace_bytes(B, Lc),
                   L.vamd_group_outcome_advantage_workspace_bytes(B, Lc, n_groups))
    ws = torch.zeros(ws_bytes, dtype=torch.uint8, device=dev)
    out = torch.empty(8, device=dev)
    coef = torch.empty(B, device=dev)
    mom = torch.empty(8, dtype=torch.float64, device=dev)
    gid = torch.arange(n_groups, device=dev).repeat_interleave(B // n_groups)
    rows_by_group = torch.arange(B, device=dev)                       # gid is already sorted
    group_offsets = torch.arange(0, B + 1, B // n_groups, device=dev)
    # scratch without arrival counters (these entry points overwrite all of it)
    ws_otb = torch.empty(max(L.vamd_otb_advantage_workspace_bytes(B, Lc, 0), L.vamd_data_metrics_workspace_bytes(B, Lc),
                             L.vamd_rollout_correction_workspace_bytes(B, Lc),
                             L.vamd_policy_loss_cov_workspace_bytes(B, Lc)), dtype=torch.uint8, device=dev)
    metrics = torch.empty(64, dtype=torch.float64, device=dev)
    attention = torch.ones(B, Lc, dtype=torch.int64, device=dev)      # no prompt columns: response part only
    st = _cabi.stream_ptr(dev)
    chk = _cabi.check
    wsp, wsn = ws.data_ptr(), ws.numel()
    none3 = (-1.0, -1.0, -1.0)   # agg_loss: batch_num_tokens, global_batch_size, loss_scale_factor not given

    def P(s, *names):
        return tuple(s[n].data_ptr() for n in names)

    def grpo(s):
        chk(L.vamd_grpo_advantage(*P(s, "a", "mask"), 0, gid.data_ptr(), B, Lc, n_groups, 1e-6, 1, 0, *P(s, "o1"), None,
                                  wsp, wsn, st))

    def policy(s, grad):
        outs = (*P(s, "o1"), coef.data_ptr()) if grad else (None, None)
        chk(L.vamd_policy_loss_forward(*P(s, "a", "b", "c", "mask"), 0, None, B, Lc, 0.2, 0.2, 3.0, 0, 1.0, *none3,
                                       out.data_ptr(), *outs, wsp, wsn, st))

    one = torch.ones(1, device=dev)

    def policy_autograd(s):   # what autograd runs: the forward kernel, then the gradient scaled by the upstream scalar
        policy(s, True)
        chk(L.vamd_scale_rows(*P(s, "o1"), coef.data_ptr(), one.data_ptr(), 1.0, B, Lc, *P(s, "o2"), st))

    def gae(s):
        chk(L.vamd_gae(*P(s, "a", "b", "mask"), 0, B, Lc, 1.0, 0.95, 1, *P(s, "o1", "o2"), mom.data_ptr(), wsp, wsn, st))

    def value(s):
        chk(L.vamd_value_loss_forward(*P(s, "a", "b", "c", "mask"), 0, B, Lc, 0.5, 0, out.data_ptr(), *P(s, "o1"),
                                      coef.data_ptr(), wsp, wsn, st))

    def kl(s):
        chk(L.vamd_kl_loss_forward(*P(s, "a", "b", "mask"), 0, B, Lc, 3, 0, 0, 1.0, *none3, out.data_ptr(), *P(s, "o1"),
                                   coef.data_ptr(), wsp, wsn, st))

    def moments(s):
        chk(L.vamd_masked_moments(*P(s, "a", "mask"), 0, B, Lc, 0, mom.data_ptr(), wsp, wsn, st))

    def otb(s):   # a: rewards, b: old log-probs, c: sum of squared probabilities
        chk(L.vamd_otb_advantage(*P(s, "a", "mask"), 0, *P(s, "b", "c"), None, rows_by_group.data_ptr(),
                                 group_offsets.data_ptr(), None, B, Lc, n_groups, 0, 1e-8, *P(s, "o1", "o2"),
                                 ws_otb.data_ptr(), ws_otb.numel(), st))

    def kl_reward(s):
        chk(L.vamd_apply_kl_penalty(*P(s, "a", "b", "c", "mask"), 0, B, Lc, 3, 0.05, *P(s, "o1"), out.data_ptr(),
                                    wsp, wsn, st))

    def data_metrics(s):
        chk(L.vamd_data_metrics(*P(s, "a", "b", "c", "o1", "o2", "mask"), 0, attention.data_ptr(), 1, B, 0, Lc,
                                metrics.data_ptr(), ws_otb.data_ptr(), ws_otb.numel(), st))

    def rollout_corr(s):
        chk(L.vamd_rollout_correction(*P(s, "a", "b", "mask"), 0, B, Lc, 1, 2.0, 0, *P(s, "o1"), metrics.data_ptr(),
                                      ws_otb.data_ptr(), ws_otb.numel(), st))

    def geo_mean(s):
        chk(L.vamd_policy_loss_variant_forward(6, *P(s, "a", "b", "c", "mask"), 0, None, B, Lc, 0.2, 0.2, 3.0, 1.0, 1.0,
                                               0, 1.0, *none3, out.data_ptr(), *P(s, "o1"), coef.data_ptr(), wsp, wsn,
                                               st))

    def gspo(s):   # variant 4, aggregated as seq-mean-token-mean (mode 2) as the reference always does
        chk(L.vamd_policy_loss_variant_forward(4, *P(s, "a", "b", "c", "mask"), 0, None, B, Lc, 0.2, 0.2, 3.0, 1.0, 1.0,
                                               2, 1.0, *none3, out.data_ptr(), *P(s, "o1"), coef.data_ptr(), wsp, wsn,
                                               st))

    def kl_cov(s):
        chk(L.vamd_policy_loss_cov_forward(0, *P(s, "a", "b", "c", "mask"), 0, None, B, Lc, 0.2, 0.2, 0.0, 0.0, 0.0002,
                                           1.0, 0, 0, 1.0, *none3, out.data_ptr(), *P(s, "o1"), coef.data_ptr(), None,
                                           ws_otb.data_ptr(), ws_otb.numel(), st))

    def copy(s):
        chk(L.vamd_copy_bytes(*P(s, "a", "o1"), 4 * BL, st))

    def sum4(s):
        chk(L.vamd_sum4(*P(s, "a", "b", "c", "mask", "o1"), BL, st))

    # name -> (algorithmic bytes per call, call)
    ops = {
        "grpo_advantage": (12 * BL, grpo),
        "policy_loss_fwd": (16 * BL, lambda s: policy(s, False)),
        "policy_loss_fwd_grad": (20 * BL, lambda s: policy(s, True)),
        "policy_loss_fwd_bwd_as_autograd_runs_it": (28 * BL, policy_autograd),   # + read the gradient, write it scaled
        "gae_scan_whiten": (28 * BL, gae),
        "value_loss_fwd_grad": (20 * BL, value),
        "kl_loss_fwd_grad": (16 * BL, kl),
        "masked_moments": (8 * BL, moments),
        "otb_advantage": (24 * BL, otb),                      # reads r, m, log-prob, sum pi^2; writes adv, returns
        "apply_kl_penalty": (20 * BL, kl_reward),
        "data_metrics": (24 * BL + 8 * BL, data_metrics),     # six fp32 tensors and the int64 attention mask
        "rollout_correction_token": (16 * BL, rollout_corr),
        "policy_loss_geo_mean_fwd_grad": (20 * BL, geo_mean),  # GMPO and GSPO: a per-sequence sum, then the per-token
        "policy_loss_gspo_fwd_grad": (20 * BL, gspo),          # pass, in one launch over the inputs where the rows allow
        "policy_loss_kl_cov_fwd_grad": (20 * BL, kl_cov),      # statistics, keys, 3 histogram passes, loss: 12 launches
        "copy_yardstick": (8 * BL, copy),
        "sum4_yardstick": (20 * BL, sum4),                    # four tensors in, one out: the traffic of a loss with gradient
    }
    res = {}
    for name, (nbytes, fn) in ops.items():
        if only is not None and name not in only:
            continue
        for s in sets:
            fn(s)
        torch.cuda.synchronize()
        reps = 48
        us = float("inf")
        for _ in range(3):   # best of three timed loops: a host hiccup between launches shows up as GPU idle time
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(reps):
                fn(sets[i % nset])
            e1.record()
            torch.cuda.synchronize()
            us = min(us, e0.elapsed_time(e1) / reps * 1e3)
        gbps = nbytes / us / 1e3
        res[name] = {"us": us, "algorithmic_bytes": nbytes, "GBps": gbps, "frac_of_8TBps": gbps / 8000.0}
    if with_cpu:
        s = {k: v.cpu() for k, v in sets[0].items()}
        idx = gid.cpu().numpy()

        def cpu_ms(fn):
            t0 = time.perf_counter()
            fn()
            return (time.perf_counter() - t0) * 1e3

        res["grpo_advantage"]["cpu_ms"] = cpu_ms(lambda: O.grpo_outcome_advantage(s["a"].clone(), s["mask"], idx))
        res["gae_scan_whiten"]["cpu_ms"] = cpu_ms(lambda: O.gae_advantage_return(s["a"], s["b"], s["mask"], 1.0, 0.95))
        res["policy_loss_fwd"]["cpu_ms"] = cpu_ms(
            lambda: O.policy_loss_vanilla(s["a"], s["b"], s["c"], s["mask"], "token-mean"))
        res["value_loss_fwd_grad"]["cpu_ms"] = cpu_ms(
            lambda: O.value_loss(s["a"], s["b"], s["c"], s["mask"], 0.5, "token-mean"))
        res["kl_loss_fwd_grad"]["cpu_ms"] = cpu_ms(
            lambda: O.agg_loss(O.kl_penalty(s["a"], s["b"], "low_var_kl"), s["mask"], "token-mean"))
        res["masked_moments"]["cpu_ms"] = cpu_ms(lambda: O.masked_var(s["a"], s["mask"]))
        res["apply_kl_penalty"]["cpu_ms"] = cpu_ms(
            lambda: O.apply_kl_penalty(s["c"], s["a"], s["b"], s["mask"], 0.05, "kl"))
        res["rollout_correction_token"]["cpu_ms"] = cpu_ms(
            lambda: (O.rollout_correction_weights(s["a"] - s["b"], s["mask"], "token", 2.0, False),
                     O.offpolicy_metrics(s["a"], s["b"], s["mask"])))
    return res


def policy_math_chain(dev, B: int = 512, Lc: int = 4096, n_groups: int = 64) -> dict:
    """GRPO advantage -> policy loss with gradient -> GAE with whitening -> value loss with gradient (one launch
    each), the per-step chain of the two policy-math benchmark configurations, launched eagerly and replayed from one captured HIP graph (microseconds
    per chain, best of three loops of 50)."""
    import torch

    from verl_amd import _cabi

    L = _cabi.lib()
    g = torch.Generator(device=dev).manual_seed(0)
    f = lambda: torch.randn(B, Lc, device=dev, generator=g)
    lens = torch.randint(64, Lc + 1, (B,), device=dev, generator=g)
    mask = (torch.arange(Lc, device=dev)[None, :] < lens[:, None]).float()
    rewards, old, values = f(), f() * 0.5 - 1, f()
    new, vpreds = old + 0.05 * f(), values + 0.5 * f()
    adv, grad, gae_adv, gae_ret, vgrad = (torch.empty(B, Lc, device=dev) for _ in range(5))
    out, coef, mom = torch.empty(4, device=dev), torch.empty(B, device=dev), torch.empty(8, dtype=torch.float64, device=dev)
    gid = torch.arange(n_groups, device=dev).repeat_interleave(B // n_groups)
    ws = torch.zeros(max(1 << 22, L.vamd_group_outcome_advantage_workspace_bytes(B, Lc, n_groups),
                         L.vamd_policy_loss_variant_workspace_bytes(B, Lc)), dtype=torch.uint8, device=dev)
    chk, P = _cabi.check, (lambda t: t.data_ptr())

    def chain():
        st = _cabi.stream_ptr(dev)
        chk(L.vamd_grpo_advantage(P(rewards), P(mask), 0, P(gid), B, Lc, n_groups, 1e-6, 1, 0, P(adv), None, P(ws),
                                  ws.numel(), st))
        chk(L.vamd_policy_loss_forward(P(old), P(new), P(adv), P(mask), 0, None, B, Lc, 0.2, 0.2, 3.0, 0, 1.0, -1.0, -1.0,
                                       -1.0, P(out), P(grad), P(coef), P(ws), ws.numel(), st))
        chk(L.vamd_gae(P(rewards), P(values), P(mask), 0, B, Lc, 1.0, 0.95, 1, P(gae_adv), P(gae_ret), P(mom), P(ws),
                       ws.numel(), st))
        chk(L.vamd_value_loss_forward(P(vpreds), P(gae_ret), P(values), P(mask), 0, B, Lc, 0.5, 0, P(out), P(vgrad),
                                      P(coef), P(ws), ws.numel(), st))

    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        chain()
    torch.cuda.current_stream(dev).wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        chain()

    def timed(fn, reps=50):
        best = float("inf")
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            best = min(best, e0.elapsed_time(e1) / reps * 1e3)
        return best

    return {"launches_per_chain": 4, "eager_us": timed(chain), "hip_graph_us": timed(graph.replay)}


def _host_profiles(ops: dict, calls: int = 1000, top: int = 14) -> dict:
    """cProfile over `calls` calls of each op: where the host time of a call goes, microseconds per call, the `top`
    entries by own time (a profiled call runs about 1.5 times slower than an unprofiled one)."""
    import cProfile
    import pstats

    import torch

    out = {}
    for name, fn in ops.items():
        for _ in range(500):   # long enough for the device to leave its idle clocks
            fn()
        torch.cuda.synchronize()
        pr = cProfile.Profile()
        t0 = time.perf_counter()
        pr.enable()
        for _ in range(calls):
            fn()
        torch.cuda.synchronize()
        pr.disable()
        wall = (time.perf_counter() - t0) / calls * 1e6
        st = pstats.Stats(pr)
        rows = []
        for (fname, line, func), (cc, nc, tt, ct, _) in st.stats.items():
            rows.append({"function": f"{os.path.basename(fname)}:{line}({func})", "calls_per_call": nc / calls,
                         "own_us": tt / calls * 1e6, "cumulative_us": ct / calls * 1e6})
        rows.sort(key=lambda r: -r["own_us"])
        out[name] = {"wall_us_per_call_profiled": wall, "top": rows[:top]}
    return out


def policy_math_python_path(dev, B: int = 512, Lc: int = 4096, n_groups: int = 64, profile: bool = False) -> dict:
    """The same operations called the way the trainer calls them -- through the functions of
    ``verl_amd.trainer.ppo.core_algos`` / ``verl_amd.utils.torch_functional`` with torch tensors on the GPU --
    so that argument checks, output allocation, ctypes marshalling and the host synchronisations the interfaces
    require (Python-float metrics) are all inside the figure: wall-clock microseconds per call over 200 calls that
    end in one device synchronisation (best of three loops)."""
    import numpy as np
    import torch

    import verl_amd.utils.torch_functional as VF
    from verl_amd.trainer.ppo import core_algos as CA

    g = torch.Generator(device=dev).manual_seed(0)
    f = lambda: torch.randn(B, Lc, device=dev, generator=g)
    lens = torch.randint(64, Lc + 1, (B,), device=dev, generator=g)
    mask = (torch.arange(Lc, device=dev)[None, :] < lens[:, None]).float()
    rewards, old, values = f(), f() * 0.5 - 1, f()
    new, vpreds = (old + 0.05 * f()).requires_grad_(), (values + 0.5 * f()).requires_grad_()
    adv, returns = f(), f()
    index = np.repeat(np.arange(n_groups), B // n_groups)

    class Cfg:
        clip_ratio, clip_ratio_low, clip_ratio_high, global_batch_info = 0.2, None, None, {}

        @staticmethod
        def get(key, default=None):
            return default

    def policy_fwd():
        with torch.no_grad():
            CA.compute_policy_loss_vanilla(old, new, adv, mask, "token-mean", Cfg)

    def policy_fwd_bwd():
        loss, _ = CA.compute_policy_loss_vanilla(old, new, adv, mask, "token-mean", Cfg)
        torch.autograd.grad(loss, new)

    def value_fwd_bwd():
        loss, _ = CA.compute_value_loss(vpreds, returns, values, mask, 0.5, "token-mean")
        torch.autograd.grad(loss, vpreds)

    def both_losses_one_backward():
        # the way an update step meets them: both losses in one graph, one backward call for the sum
        pl, _ = CA.compute_policy_loss_vanilla(old, new, adv, mask, "token-mean", Cfg)
        vl, _ = CA.compute_value_loss(vpreds, returns, values, mask, 0.5, "token-mean")
        torch.autograd.grad(pl + 0.5 * vl, (new, vpreds))

    ops = {
        "grpo_advantage": lambda: CA.compute_grpo_outcome_advantage(rewards, mask, index),
        "policy_loss_fwd": policy_fwd,
        "policy_loss_fwd_grad": policy_fwd_bwd,
        "gae_scan_whiten": lambda: CA.compute_gae_advantage_return(rewards, values, mask, 1.0, 0.95),
        "value_loss_fwd_grad": value_fwd_bwd,
        "policy_and_value_loss_one_backward": both_losses_one_backward,
        "masked_mean": lambda: VF.masked_mean(values, mask),
        "masked_whiten": lambda: VF.masked_whiten(values, mask),
        "agg_loss_token_mean": lambda: CA.agg_loss(values, mask, "token-mean"),
    }
    if profile:
        return _host_profiles({k: ops[k] for k in ("policy_loss_fwd", "policy_loss_fwd_grad", "value_loss_fwd_grad",
                                                   "policy_and_value_loss_one_backward")})
    res = {}
    for name, fn in ops.items():
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(3):
            t0 = time.perf_counter()
            for _ in range(200):
                fn()
            torch.cuda.synchronize()
            best = min(best, (time.perf_counter() - t0) / 200 * 1e6)
        res[name] = {"us_per_call": best}
    return res


def _read_sclk_mhz():
    """Current shader clock in MHz from the driver's sysfs table (the line marked '*'), or None."""
    import glob

    for path in sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")):
        try:
            for ln in open(path).read().splitlines():
                if ln.rstrip().endswith("*"):
                    digits = "".join(c for c in ln.split(":", 1)[1] if c.isdigit())
                    if digits:
                        return int(digits)
        except (OSError, IndexError):
            continue
    return None


def _read_power_w():
    """Board power in watts as the driver reports it (hwmon power1_input, microwatts), and the cap; (None, None) if
    unreadable."""
    import glob

    for path in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input")):
        try:
            watts = int(open(path).read().strip()) / 1e6
            cap = None
            try:
                cap = int(open(path.replace("power1_input", "power1_cap")).read().strip()) / 1e6
            except (OSError, ValueError):
                pass
            return watts, cap
        except (OSError, ValueError):
            continue
    return None, None


def _sclk_sampler():
    """Background reader of the shader clock, for the ceiling probe: returns (stop, samples).  Reads sysfs, starts no
    other program."""
    import threading

    samples, stop = [], threading.Event()

    def run():
        while not stop.is_set():
            mhz = _read_sclk_mhz()
            if mhz:
                samples.append((time.time(), mhz, _read_power_w()[0]))
            stop.wait(0.05)

    th = threading.Thread(target=run, daemon=True)
    th.start()
    return stop, samples


def mfma_ceiling_probe(dev, n: int, h: int, v: int, seconds: float = 1.5) -> dict:
    """Where the matrix pipes top out on THIS board and data: the head's forward kernel and the vendor GEMM
    (torch.matmul -> hipBLASLt) at the three operand layouts of the step (logits NT, d_hidden NN, d_weight TN,
    one 16384-column vocabulary chunk each), on all-zero operands and on the benchmark's random operands, each run
    back to back for `seconds` with the shader clock read beside it.  Zeros draw the least power, so the clock
    stays at its maximum there; the random figures are what power management leaves."""
    import torch

    from verl_amd import _cabi

    L = _cabi.lib()
    st = _cabi.stream_ptr(dev)
    g = torch.Generator(device=dev).manual_seed(0)
    labels = torch.randint(0, v, (n,), device=dev, generator=g)
    outs = [torch.empty(n, device=dev) for _ in range(4)]
    ws = torch.empty(L.vamd_lce_forward_workspace_bytes(n, h, v), dtype=torch.uint8, device=dev)
    vc = 16384
    stop, samples = _sclk_sampler()
    res = {}

    def run_for(fn, flops):
        fn()
        torch.cuda.synchronize()
        t_begin = time.time()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        reps = 0
        e0.record()
        while time.time() - t_begin < seconds:
            for _ in range(4):
                fn()
            reps += 4
            torch.cuda.synchronize()
        e1.record()
        torch.cuda.synchronize()
        t_end = time.time()
        ms = e0.elapsed_time(e1) / reps
        late = [(m, p) for (t, m, p) in samples if t_begin + 0.4 * (t_end - t_begin) <= t <= t_end]
        clk = [m for m, _ in late]
        pw = [p for _, p in late if p is not None]
        return {"ms": ms, "PFLOPs": flops / ms / 1e12, "sclk_MHz": (sum(clk) / len(clk)) if clk else None,
                "board_W": (sum(pw) / len(pw)) if pw else None}

    for kind in ("zeros", "random"):
        if kind == "zeros":
            hid = torch.zeros(n, h, device=dev, dtype=torch.bfloat16)
            w = torch.zeros(v, h, device=dev, dtype=torch.bfloat16)
        else:
            hid = torch.randn(n, h, device=dev, generator=g).bfloat16()
            w = (torch.randn(v, h, device=dev, generator=g) * 0.02).bfloat16()

        def fwd():
            _cabi.check(L.vamd_lce_forward(hid.data_ptr(), w.data_ptr(), labels.data_ptr(), n, h, v, 1.0,
                                           *(o.data_ptr() for o in outs), None, None, ws.data_ptr(), ws.numel(), st))

        wc = w[:vc]
        z = torch.empty(n, vc, device=dev, dtype=torch.bfloat16)
        dh = torch.empty(n, h, device=dev, dtype=torch.bfloat16)
        dw = torch.empty(vc, h, device=dev, dtype=torch.bfloat16)
        res[kind] = {
            "lce_forward_kernel": run_for(fwd, 2.0 * n * v * h),
            "vendor_gemm_NT_logits": run_for(lambda: torch.matmul(hid, wc.t(), out=z), 2.0 * n * vc * h),
        }
        if kind == "random":
            z.normal_(generator=g)
        res[kind]["vendor_gemm_NN_d_hidden"] = run_for(lambda: torch.matmul(z, wc, out=dh), 2.0 * n * vc * h)
        res[kind]["vendor_gemm_TN_d_weight"] = run_for(lambda: torch.matmul(z.t(), hid, out=dw), 2.0 * n * vc * h)
        del hid, w, wc, z, dh, dw
        # the matrix instruction alone, operands in registers: what is left of the peak when nothing moves data
        wgs, iters = 256, 4000
        if kind == "zeros":
            seed = torch.zeros(wgs * 512 * 32, dtype=torch.int32, device=dev)
        else:   # bf16 pairs with exponents near 1 and random signs / mantissas
            lo = torch.randint(0, 1 << 16, (wgs * 512 * 32,), device=dev, generator=g, dtype=torch.int32)
            hi = torch.randint(0, 1 << 16, (wgs * 512 * 32,), device=dev, generator=g, dtype=torch.int32)
            seed = ((lo & 0x80FF) | 0x3F00) | (((hi & 0x80FF) | 0x3F00) << 16)
        sink = torch.empty(wgs * 512, device=dev)
        for shape, name in ((0, "mfma_only_32x32x16"), (1, "mfma_only_16x16x32")):
            flops = float(L.vamd_mfma_yardstick_flops(shape, wgs, iters))
            res[kind][name] = run_for(
                lambda: _cabi.check(L.vamd_mfma_yardstick(shape, seed.data_ptr(), sink.data_ptr(), wgs, iters, st)), flops)
        del seed, sink
    # The other two head shapes of the configuration list, forward kernel and vendor NT GEMM over the whole
    # vocabulary, zeros against random operands: whether the clock (power) or the pipeline (stalls) holds them back.
    for name, (n2, h2, v2) in (("qwen0.5b_head_2048x896x151936", (2048, 896, 151936)),
                               ("llama8b_chunk_8192x4096x128256", (8192, 4096, 128256))):
        lab2 = torch.randint(0, v2, (n2,), device=dev, generator=g)
        outs2 = [torch.empty(n2, device=dev) for _ in range(4)]
        ws2 = torch.empty(L.vamd_lce_forward_workspace_bytes(n2, h2, v2), dtype=torch.uint8, device=dev)
        z2 = torch.empty(n2, v2, device=dev, dtype=torch.bfloat16)
        res[name] = {}
        for kind in ("zeros", "random"):
            if kind == "zeros":
                hid = torch.zeros(n2, h2, device=dev, dtype=torch.bfloat16)
                w = torch.zeros(v2, h2, device=dev, dtype=torch.bfloat16)
            else:
                hid = torch.randn(n2, h2, device=dev, generator=g).bfloat16()
                w = (torch.randn(v2, h2, device=dev, generator=g) * 0.02).bfloat16()

            def fwd2():
                _cabi.check(L.vamd_lce_forward(hid.data_ptr(), w.data_ptr(), lab2.data_ptr(), n2, h2, v2, 1.0,
                                               *(o.data_ptr() for o in outs2), None, None, ws2.data_ptr(), ws2.numel(),
                                               st))

            res[name][kind] = {
                "lce_forward_kernel": run_for(fwd2, 2.0 * n2 * v2 * h2),
                "vendor_gemm_NT_logits": run_for(lambda: torch.matmul(hid, w.t(), out=z2), 2.0 * n2 * v2 * h2),
            }
            del hid, w
        del lab2, outs2, ws2, z2
    stop.set()
    res["board_power_cap_W"] = _read_power_w()[1]
    res["note"] = ("ms per call; PFLOP/s on 2*M*N*K; sclk and board power from the driver's sysfs files over the second "
                   "half of each run (None when they cannot be read); vendor GEMMs on one 16384-column vocabulary chunk; "
                   "mfma_only_*: the bf16 matrix instruction of that shape in a register-only loop, 8 wavefronts per CU")
    return res


def time_head_mode(step, steps: int, warmup: int, n: int, dev) -> dict:
    """Wall-clock milliseconds per forward+backward step and the peak device memory the step adds."""
    import torch

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats(dev)
    base = torch.cuda.memory_allocated(dev)
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    return {"ms_per_step": dt / steps * 1e3, "tokens_per_s": n * steps / dt,
            "peak_step_memory_bytes": torch.cuda.max_memory_allocated(dev) - base}


def head_kernel_times(L, step, prof_steps: int) -> dict:
    """Per-kernel durations from HIP events recorded on the launch stream around every head kernel launch."""
    from verl_amd import _cabi

    L.vamd_lce_timing_enable(1)
    for _ in range(prof_steps):
        step()
    ms = (ctypes.c_double * len(KERNEL_NAMES))()
    cnt = (ctypes.c_int64 * len(KERNEL_NAMES))()
    _cabi.check(L.vamd_lce_timing_collect(ms, cnt))
    L.vamd_lce_timing_enable(0)
    kernels = {}
    for i, name in enumerate(KERNEL_NAMES):
        if cnt[i]:
            kernels[name] = {"ms_per_step": ms[i] / prof_steps, "launches_per_step": cnt[i] / prof_steps,
                             "avg_ms": ms[i] / cnt[i]}
    return kernels


def composed_actor_step(dev, steps: int) -> dict:
    """One actor update step the way the trainer composes it, at the benchmark's head shape as 4 sequences of 4096
    tokens: head -> per-token log-prob and entropy -> clipped policy loss + entropy bonus + KL loss -> one backward
    through everything.  Beside it the same step with the three losses replaced by plain sums of the head's outputs:
    the difference is what the losses cost inside a step (kernels, their Python mirror and their share of autograd),
    where called alone a loss with its backward pays a whole autograd launch of its own."""
    import types

    import torch

    from verl_amd.trainer.ppo import core_algos as CA
    from verl_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy

    B, Lc, h, v = 4, 4096, 3584, 152064
    n = B * Lc
    g = torch.Generator(device=dev).manual_seed(9)
    hidden = torch.randn(n, h, device=dev, generator=g).bfloat16().requires_grad_()
    weight = (torch.randn(v, h, device=dev, generator=g) * 0.02).bfloat16().requires_grad_()
    labels = torch.randint(0, v, (n,), device=dev, generator=g)
    lens = torch.randint(Lc // 2, Lc + 1, (B,), device=dev, generator=g)
    mask = (torch.arange(Lc, device=dev)[None, :] < lens[:, None]).float()
    adv = torch.randn(B, Lc, device=dev, generator=g)
    cfg = types.SimpleNamespace(clip_ratio=0.2, clip_ratio_low=None, clip_ratio_high=None, global_batch_info={})
    cfg.get = lambda k, d=None: getattr(cfg, k, d)
    with torch.no_grad():
        old_lp, _ = linear_cross_entropy(hidden, weight, labels, 1.0)
        old_lp = old_lp.view(B, Lc) + 0.05 * torch.randn(B, Lc, device=dev, generator=g)
        ref_lp = old_lp + 0.05 * torch.randn(B, Lc, device=dev, generator=g)

    def with_losses():
        lp, ent = linear_cross_entropy(hidden, weight, labels, 1.0)
        lp, ent = lp.view(B, Lc), ent.view(B, Lc)
        pg, _ = CA.compute_policy_loss_vanilla(old_lp, lp, adv, mask, "token-mean", cfg)
        loss = pg - 0.001 * CA.agg_loss(ent, mask, "token-mean") + 0.01 * CA.compute_kl_loss(lp, ref_lp, mask)
        torch.autograd.grad(loss, (hidden, weight))

    def plain_sums():
        lp, ent = linear_cross_entropy(hidden, weight, labels, 1.0)
        torch.autograd.grad((lp * mask.view(-1)).sum() - 0.001 * (ent * mask.view(-1)).sum(), (hidden, weight))

    def timed(fn):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3

    a, b = timed(with_losses), timed(plain_sums)
    return {"batch": B, "response_length": Lc, "hidden_size": h, "vocab": v, "ms_with_policy_entropy_kl_losses": a,
            "ms_with_plain_sums_instead": b, "losses_share_ms": a - b}


def other_head_configs(dev, steps: int, with_cpu: bool = True) -> dict:
    """BASELINE configs[0] (Qwen2.5-0.5B head shape, forward only) and configs[4] (Llama-3-8B head shape, 65536
    tokens as eight 8192-token chunks, T = 0.7, entropy coefficient folded into the backward, weight gradient summed
    over the chunks in fp32), timed end to end through the host mirror."""
    import torch

    from verl_amd.utils.kernel import linear_cross_entropy as K

    g = torch.Generator(device=dev).manual_seed(3)
    res = {}
    n, h, v = 2048, 896, 151936
    hid = torch.randn(n, h, device=dev, generator=g).bfloat16()
    w = (torch.randn(v, h, device=dev, generator=g) * 0.02).bfloat16()
    lab = torch.randint(0, v, (n,), device=dev, generator=g)

    def timed(fn, reps):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps * 1e3

    with torch.no_grad():
        ms = timed(lambda: K.linear_cross_entropy(hid, w, lab, 1.0), 20)
    res["qwen0.5b_forward_only"] = {"n_tokens": n, "hidden_size": h, "vocab": v, "ms": ms, "tokens_per_s": n / ms * 1e3,
                                    "PFLOPs_algorithmic": 2.0 * n * v * h / ms / 1e12}
    if with_cpu:   # this configuration is small enough to run in full on the host: the oracle's chunked torch backend
        import oracle as O

        torch.set_num_threads(os.cpu_count() or 1)
        hc, wc, lc = hid.cpu(), w.cpu(), lab.cpu()
        t0 = time.perf_counter()
        with torch.no_grad():
            O.fused_linear_for_ppo_chunked(hc, wc, lc, 1.0, 512)
        dt = time.perf_counter() - t0
        res["qwen0.5b_forward_only"]["cpu_baseline"] = {
            "value": n / dt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"all {n} tokens, chunked torch backend, bf16 GEMMs, forward once, {dt:.2f} s"}
        del hc, wc, lc
    del hid, w, lab
    n, h, v, T, chunk = 65536, 4096, 128256, 0.7, 8192
    hid = torch.randn(n, h, device=dev, generator=g).bfloat16()
    w = (torch.randn(v, h, device=dev, generator=g) * 0.02).bfloat16()
    lab = torch.randint(0, v, (n,), device=dev, generator=g)
    g_lp = torch.randn(n, device=dev, generator=g)
    acc32 = torch.empty(v, h, device=dev, dtype=torch.float32)
    d_weight = torch.empty_like(w)
    n_chunks = n // chunk

    def long_rollout():
        for ci in range(n_chunks):
            sl = slice(ci * chunk, (ci + 1) * chunk)
            _, _, lse, mz = K.efficient_entropy_forward(hid[sl], w, lab[sl], 0, T)
            K.efficient_entropy_backward(g_lp[sl], None, hid[sl], w, lab[sl], lse, mz, 0, T, d_entropy_scalar=0.001,
                                         d_weight_acc32=acc32, d_weight_out=d_weight,
                                         acc32_step="first" if ci == 0 else ("last" if ci == n_chunks - 1 else "middle"))

    ms = timed(long_rollout, max(1, min(steps, 3)))
    res["llama8b_long_rollout_fwd_bwd"] = {"n_tokens": n, "hidden_size": h, "vocab": v, "temperature": T,
                                           "token_chunk": chunk, "ms": ms, "tokens_per_s": n / ms * 1e3,
                                           "PFLOPs_algorithmic": 6.0 * n * v * h / ms / 1e12,
                                           "mode": "recompute, fp32 d_weight accumulation over the 8 chunks"}
    return res


def unfused_logits_rates(dev) -> dict:
    """The per-token definitions on materialised logits (row-wise online softmax): microseconds, algorithmic bytes
    (the logits once forward; logits in + gradient out backward) and the fraction of 8 TB/s, at 4096 tokens of the
    Qwen2.5-7B vocabulary.  Two buffer sets alternate so that a call never finds its rows in the Infinity Cache."""
    import torch

    from verl_amd import _cabi

    L = _cabi.lib()
    n, v = 4096, 152064
    st = _cabi.stream_ptr(dev)
    res = {}
    for name, dtype, code, esz in (("bf16", torch.bfloat16, 1, 2), ("fp32", torch.float32, 0, 4)):
        sets = [torch.randn(n, v, device=dev, dtype=dtype) for _ in range(2)]
        grads = [torch.empty(n, v, device=dev, dtype=dtype) for _ in range(2)]
        labels = torch.randint(0, v, (n,), device=dev)
        f = [torch.empty(n, device=dev) for _ in range(4)]
        g_lp = torch.randn(n, device=dev)

        def fwd(i):
            _cabi.check(L.vamd_row_softmax_stats(sets[i].data_ptr(), code, n, v, v, labels.data_ptr(), f[0].data_ptr(),
                                                 f[1].data_ptr(), f[2].data_ptr(), f[3].data_ptr(), st))

        def bwd(i):
            _cabi.check(L.vamd_row_softmax_backward(sets[i].data_ptr(), code, n, v, v, labels.data_ptr(), f[2].data_ptr(),
                                                    f[3].data_ptr(), g_lp.data_ptr(), g_lp.data_ptr(),
                                                    grads[i].data_ptr(), v, st))

        for label, fn, nbytes in (("forward", fwd, n * v * esz), ("backward", bwd, 2 * n * v * esz)):
            fn(0); fn(1)
            torch.cuda.synchronize()
            best = float("inf")
            for _ in range(3):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for i in range(8):
                    fn(i % 2)
                e1.record()
                torch.cuda.synchronize()
                best = min(best, e0.elapsed_time(e1) / 8 * 1e3)
            res[f"{name}_{label}"] = {"us": best, "algorithmic_bytes": nbytes, "GBps": nbytes / best / 1e3,
                                      "frac_of_8TBps": nbytes / best / 1e3 / 8000.0}
        del sets, grads
    res["shape"] = {"n_tokens": n, "vocab": v}
    return res


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--cpu-tokens", type=int, default=8192, help="token sample for the CPU baseline (0 = skip)")
    ap.add_argument("--head-only", action="store_true",
                    help="only the headline workload and its per-kernel timing (what the profiler runs trace)")
    ap.add_argument("--ceiling-only", action="store_true",
                    help="only the matrix-pipe ceiling probe (zeros against random operands, vendor GEMMs beside "
                         "the forward kernel): what a counter pass for the shader clock runs")
    ap.add_argument("--ceiling-seconds", type=float, default=1.5, help="how long the probe keeps each kernel running")
    ap.add_argument("--python-path-profile", action="store_true",
                    help="only a cProfile table of the Python mirror's loss calls (host time per call)")
    ap.add_argument("--policy-math-only", action="store_true",
                    help="only the [B, L] kernels at B = 2048, L = 16384 after the 1 GiB copy: what a counter pass for "
                         "their memory traffic runs")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: --gpus {args.gpus} is not supported (every box here has one GPU; "
              "across GPUs the path shards by tokens and needs no collective in its forward pass)", file=sys.stderr)
        sys.exit(2)

    import torch

    from verl_amd import _cabi
    from verl_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy, logits_cache_budget_bytes

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    n, h, v, T = 16384, 3584, 152064, 1.0
    if args.ceiling_only:
        print(json.dumps({"mfma_ceiling_probe": mfma_ceiling_probe(dev, n, h, v, seconds=args.ceiling_seconds)}))
        return
    if args.python_path_profile:
        print(json.dumps({"python_path_host_profile_b512_l4096": policy_math_python_path(dev, profile=True)}))
        return
    if args.policy_math_only:
        a = torch.empty(1 << 30, dtype=torch.uint8, device=dev)   # the copy the counters are scaled by
        b = torch.empty_like(a)
        _cabi.check(_cabi.lib().vamd_copy_bytes(a.data_ptr(), b.data_ptr(), a.numel(), _cabi.stream_ptr(dev)))
        torch.cuda.synchronize()
        del a, b
        only = {"grpo_advantage", "policy_loss_fwd", "policy_loss_fwd_grad", "gae_scan_whiten", "value_loss_fwd_grad",
                "kl_loss_fwd_grad", "masked_moments", "apply_kl_penalty", "data_metrics"}
        print(json.dumps({"policy_math_b2048_l16384": policy_math_rates(dev, with_cpu=False, B=2048, Lc=16384,
                                                                         n_groups=256, only=only)}))
        return
    g = torch.Generator(device=dev).manual_seed(0)
    hidden = torch.randn(n, h, device=dev, generator=g).bfloat16().requires_grad_()
    weight = (torch.randn(v, h, device=dev, generator=g) * 0.02).bfloat16().requires_grad_()
    labels = torch.randint(0, v, (n,), device=dev, generator=g)
    g_lp = torch.randn(n, device=dev, generator=g)
    g_ent = torch.full((n,), 0.001, device=dev)

    def step():
        lp, ent = linear_cross_entropy(hidden, weight, labels, T)
        return torch.autograd.grad((lp, ent), (hidden, weight), (g_lp, g_ent))

    # one plain 1 GiB copy, untimed: under a counter-collecting profiler its FETCH_SIZE / WRITE_SIZE
    # readings are the yardstick that turns the other kernels' readings into bytes
    L = _cabi.lib()
    src = torch.empty(COPY_YARDSTICK_BYTES, dtype=torch.uint8, device=dev).random_(0, 256)
    dst = torch.empty_like(src)
    _cabi.check(L.vamd_copy_bytes(src.data_ptr(), dst.data_ptr(), COPY_YARDSTICK_BYTES, _cabi.stream_ptr(dev)))
    torch.cuda.synchronize()
    del src, dst

    # The headline is the mode the library ships as its default (whatever VAMD_LCE_LOGITS_CACHE_GB says in this
    # process's environment; unset = no cache, the backward pass recomputes the logits).
    default_cached = 4 * n * v <= logits_cache_budget_bytes()
    head = time_head_mode(step, args.steps, args.warmup, n, dev)
    ms_per_step, tokens_per_s = head["ms_per_step"], head["tokens_per_s"]
    prof_steps = max(1, min(args.steps, 5))
    kernels = head_kernel_times(L, step, prof_steps)

    gemm_flops = 2.0 * n * v * h
    peak = PEAK_BF16_TFLOPS * 1e12

    def fractions(ms, cached):
        return {"step_algorithmic_frac": 6.0 * gemm_flops / 2.0 / (ms * 1e-3) / peak,
                "step_hardware_frac": (6.0 if cached else 8.0) * gemm_flops / 2.0 / (ms * 1e-3) / peak}

    dom = max((k for k in kernels if k in GEMMS_PER_STEP), key=lambda k: kernels[k]["ms_per_step"])
    d = kernels[dom]
    flops_per_launch = GEMMS_PER_STEP[dom] * gemm_flops / d["launches_per_step"]
    achieved = flops_per_launch / (d["avg_ms"] * 1e-3) / 1e12
    roofline = {
        "bound": "mfma",
        "kernel": dom,
        "achieved": achieved,
        "peak": PEAK_BF16_TFLOPS,
        "unit": "TFLOP/s",
        "frac": achieved / PEAK_BF16_TFLOPS,
        "traffic": measured_traffic(dom)[0],
        "traffic_measured_at_commit": measured_traffic(dom)[1],
        "flops_per_launch": flops_per_launch,
        "avg_launch_ms": d["avg_ms"],
        **fractions(ms_per_step, default_cached),
        "kernels": kernels,
    }

    # the other mode beside it, same process, same tensors
    modes = {}
    this_mode = "logits_cache" if default_cached else "recompute"
    modes[this_mode] = {**head, **fractions(ms_per_step, default_cached), "default": True}
    saved_env = os.environ.get("VAMD_LCE_LOGITS_CACHE_GB")
    os.environ["VAMD_LCE_LOGITS_CACHE_GB"] = "0" if default_cached else "16"
    other = time_head_mode(step, args.steps, args.warmup, n, dev)
    other_kernels = head_kernel_times(L, step, prof_steps)
    modes["recompute" if default_cached else "logits_cache"] = {
        **other, **fractions(other["ms_per_step"], not default_cached), "default": False,
        "kernels": other_kernels,
        "enable": "VAMD_LCE_LOGITS_CACHE_GB=0" if default_cached else "VAMD_LCE_LOGITS_CACHE_GB=16"}
    if saved_env is None:
        del os.environ["VAMD_LCE_LOGITS_CACHE_GB"]
    else:
        os.environ["VAMD_LCE_LOGITS_CACHE_GB"] = saved_env

    # One-sided steps in the default mode: the backward runs only the gradient GEMM of the input that requires a
    # gradient (a frozen head / LoRA on the trunk; or a head fine-tuned on detached hidden states).
    def one_sided(wrt):
        h = hidden if wrt is hidden else hidden.detach()   # the frozen input does not require a gradient
        w = weight if wrt is weight else weight.detach()

        def run():
            lp, ent = linear_cross_entropy(h, w, labels, T)
            return torch.autograd.grad((lp, ent), (wrt,), (g_lp, g_ent))
        return run

    for key, wrt, what in (("frozen_weight", hidden, "d_hidden only"), ("frozen_hidden", weight, "d_weight only")):
        r = time_head_mode(one_sided(wrt), args.steps, args.warmup, n, dev)
        hw_gemms = 2.0 if default_cached else 3.0     # forward + (recompute) + one gradient GEMM
        modes[key] = {**r, "default": False, "gradients": what,
                      "step_algorithmic_frac": 2.0 * gemm_flops / (r["ms_per_step"] * 1e-3) / peak,
                      "step_hardware_frac": hw_gemms * gemm_flops / (r["ms_per_step"] * 1e-3) / peak,
                      "kernels": head_kernel_times(L, one_sided(wrt), prof_steps)}

    # The same step with the upstream gradients of 40 % of the tokens zero, in runs (prompt tokens between responses,
    # which the loss masks out): the backward kernels run over the other tokens only.  Beside it the same gradients
    # with that switched off.
    keep = (torch.arange(n, device=dev) % 2048) >= 820          # 820 prompt tokens in every 2048
    g_lp_masked, g_ent_masked = g_lp * keep, g_ent * keep

    def masked_step():
        lp, ent = linear_cross_entropy(hidden, weight, labels, T)
        return torch.autograd.grad((lp, ent), (hidden, weight), (g_lp_masked, g_ent_masked))

    saved_skip = os.environ.get("VAMD_LCE_SKIP_ZERO_GRAD_TOKENS")
    masked = {}
    import verl_amd.utils.kernel.linear_cross_entropy as head_module
    for key, flag in (("active_tokens_only", "1"), ("all_tokens", "0")):
        os.environ["VAMD_LCE_SKIP_ZERO_GRAD_TOKENS"] = flag
        head_module._ACTIVE_PROBE["rest"] = 0   # the steps before found every token active: look again now
        r = time_head_mode(masked_step, args.steps, args.warmup, n, dev)
        masked[key] = {"ms_per_step": r["ms_per_step"], "tokens_per_s": r["tokens_per_s"]}
    if saved_skip is None:
        del os.environ["VAMD_LCE_SKIP_ZERO_GRAD_TOKENS"]
    else:
        os.environ["VAMD_LCE_SKIP_ZERO_GRAD_TOKENS"] = saved_skip
    modes["prompt_tokens_masked_40pct"] = {**masked, "default": False,
                                           "zero_gradient_tokens": int(n - int(keep.sum())), "of_tokens": n}

    line = {
        "metric": "tokens/s fwd+bwd logprob+entropy head @Qwen2.5-7B shape; MFMA util %",
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "fused log-prob+entropy head forward+backward, Qwen2.5-7B head shape "
                               "(BASELINE configs[1])",
                   "n_tokens": n, "hidden_size": h, "vocab": v, "temperature": T,
                   "upstream": "dlogprob ~ N(0,1) fp32, dentropy = 0.001",
                   "backward": "logits cache" if default_cached else "recomputes the logits (no [tokens, vocab] tensor)",
                   "fp32_logits_cache_bytes": 4 * n * v if default_cached else 0},
        # algorithmic-or-recompute flops of the step over the 2.5 PFLOP/s peak: what share of the matrix pipes' peak
        # the step's own arithmetic amounts to.  It is not a hardware counter.
        "step_hardware_flops_pct_of_peak": 100.0 * roofline["step_hardware_frac"],
        "roofline": roofline,
        "head_modes": modes,
    }
    if args.head_only:
        print(json.dumps(line))
        return

    line["cpu_baseline"] = cpu_baseline(args.cpu_tokens, h, v, T) if args.cpu_tokens > 0 else None
    del hidden, weight
    torch.cuda.empty_cache()
    line["mfma_ceiling_probe"] = mfma_ceiling_probe(dev, n, h, v, seconds=args.ceiling_seconds)
    torch.cuda.empty_cache()
    line["head_other_configs"] = other_head_configs(dev, args.steps, with_cpu=args.cpu_tokens > 0)
    torch.cuda.empty_cache()
    line["actor_step_composed_b4_l4096"] = composed_actor_step(dev, args.steps)
    torch.cuda.empty_cache()
    line["unfused_logits_rows"] = unfused_logits_rates(dev)
    torch.cuda.empty_cache()
    line["policy_math_b512_l4096"] = policy_math_rates(dev, with_cpu=args.cpu_tokens > 0)
    resident = policy_math_rates(dev, with_cpu=False, buffer_sets=1,
                                 only={"grpo_advantage", "policy_loss_fwd", "policy_loss_fwd_grad", "gae_scan_whiten",
                                       "value_loss_fwd_grad", "kl_loss_fwd_grad", "masked_moments", "copy_yardstick",
                                       "sum4_yardstick"})
    line["policy_math_b512_l4096_cache_resident_us"] = {k: v["us"] for k, v in resident.items()}
    line["policy_math_python_path_b512_l4096"] = policy_math_python_path(dev)
    # the same kernels on 16 x larger tensors, where the fixed ~8 us of the single-launch reduction no longer dominates
    line["policy_math_b2048_l16384"] = policy_math_rates(dev, with_cpu=False, B=2048, Lc=16384, n_groups=256)
    line["policy_math_chain_b512_l4096"] = policy_math_chain(dev)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
