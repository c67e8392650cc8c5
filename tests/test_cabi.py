"""CPU-side checks of the boundary: the shared library loads, exports every symbol that
include/verl_amd.h declares, answers its size queries, and the host wrappers refuse to run
without a GPU instead of falling back."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from verl_amd import _cabi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "verl_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vamd_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_cabi.lib_path()):
        from verl_amd.csrc.build import build
        build(verbose=False)
    return _cabi.load_library()


def test_every_declared_symbol_is_exported_and_bound(lib):
    declared = _declared_symbols()
    assert len(declared) >= 20
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/verl_amd.h but not exported"
    assert sorted(_cabi.SIGNATURES) == declared, "ctypes prototypes and header disagree"
    assert lib.vamd_abi_version() == _cabi.ABI_VERSION
    header = open(os.path.join(os.path.dirname(__file__), "..", "include", "verl_amd.h")).read()
    assert f"#define VAMD_ABI_VERSION {_cabi.ABI_VERSION}\n" in header


def test_workspace_queries(lib):
    assert lib.vamd_lce_forward_workspace_bytes(16384, 3584, 152064) > 0
    assert lib.vamd_lce_forward_workspace_bytes(0, 3584, 152064) == 0
    n, h, v = 16384, 3584, 152064
    full = lib.vamd_lce_backward_workspace_bytes(n, h, v, 0)
    assert full < 1 << 30                                         # d_logits panel + fp32 d_hidden accumulator
    one = lib.vamd_lce_backward_workspace_bytes(256, 128, 1024, 0)
    assert one == 256 * (1024 + 128) * 2                          # a single padded panel, no accumulator
    # single-launch reductions: arrival counters (VAMD_TICKET_BYTES) + one record of doubles per 4096-column chunk
    # + 64 records for the share totals of the two-level sum
    ticket = 16640
    assert lib.vamd_masked_moments_workspace_bytes(512, 4096) == ticket + (512 + 64) * 4 * 8
    assert lib.vamd_policy_loss_workspace_bytes(512, 4097) == ticket + (512 * 2 + 64) * 5 * 8
    assert lib.vamd_gae_workspace_bytes(512, 4096) >= ticket + 512 * 4 * 8


def test_argument_errors_are_reported_without_touching_the_gpu(lib):
    rc = lib.vamd_lce_forward(None, None, None, 16, 100, 128, 1.0, None, None, None, None, None, None, None, 0, None)
    assert rc == -1 and b"multiple of 128" in lib.vamd_last_error()
    rc = lib.vamd_policy_loss_forward(None, None, None, None, 0, None, 4, 4, 0.2, 0.2, 3.0, 0, 1.0, -1.0, -1.0, -1.0,
                                      None, None, None, None, 0, None)
    assert rc == -1 and b"null pointer" in lib.vamd_last_error()


@pytest.mark.skipif(torch.cuda.is_available(), reason="needs a machine without a GPU")
def test_no_cpu_fallback():
    from verl_amd.trainer.ppo import core_algos as CA
    from verl_amd.utils import torch_functional as F
    x = torch.ones(2, 4)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        F.masked_mean(x, x)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        CA.compute_gae_advantage_return(x, x, x, 1.0, 1.0)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        CA.agg_loss(x, x, "token-mean")


def test_missing_library_fails_loudly(tmp_path):
    with pytest.raises(RuntimeError, match="is missing"):
        _cabi.load_library(str(tmp_path / "libverl_amd.so"))


def test_registries_and_host_logic_without_gpu():
    from verl_amd.trainer.ppo import core_algos as CA
    from verl_amd.utils.groupwise import as_torch_index, contiguous_group_ids
    from verl_amd.utils.kernel.linear_cross_entropy import get_entropy_reduction_enum_number
    assert CA.get_adv_estimator_fn("gae") is CA.compute_gae_advantage_return
    assert CA.get_adv_estimator_fn(CA.AdvantageEstimator.GRPO) is CA.compute_grpo_outcome_advantage
    assert CA.get_policy_loss_fn("vanilla") is CA.compute_policy_loss_vanilla
    with pytest.raises(ValueError, match="Unsupported loss mode"):
        CA.get_policy_loss_fn("gspo-not-here")
    with pytest.raises(ValueError, match="Unknown advantage estimator"):
        CA.get_adv_estimator_fn("nope")
    with pytest.raises(ValueError, match="already been registered"):
        CA.register_adv_est("grpo")(lambda: None)
    with pytest.raises(ValueError, match="Invalid loss_agg_mode"):
        CA.agg_loss(torch.ones(1, 1), torch.ones(1, 1), "bad-mode")
    assert [get_entropy_reduction_enum_number(r) for r in ("none", "sum", "mean")] == [0, 1, 2]
    with pytest.raises(ValueError, match="Invalid reduction"):
        get_entropy_reduction_enum_number("max")
    g = as_torch_index(["a", "b", "a", "c", "0042", 42])
    assert g.tolist()[4] != g.tolist()[5] and len(torch.unique(g)) == 5
    assert as_torch_index(["5", "6", "5"]).tolist() == [5, 6, 5]
    assert as_torch_index(torch.tensor([1.0, 2.0, 1.0])).tolist() == [1, 2, 1]
    assert as_torch_index(np.array([3, 3, 7])).tolist() == [3, 3, 7]
    assert as_torch_index(np.array([True, False])).tolist() == [1, 0]
    assert as_torch_index(np.array([1.5, 2.5, 1.5])).tolist() == [1, 2, 1]          # numpy floats: integer cast
    t = as_torch_index(torch.tensor([1.5, 2.5, 1.5]))                               # tensor floats: opaque labels
    assert t.tolist() == [0, 1, 0]
    ids, G = contiguous_group_ids([10, 10, 7, 99])                                  # a list: ids by first appearance
    assert G == 3 and ids.tolist() == [0, 0, 1, 2]
    ids, G = contiguous_group_ids(np.array([10, 10, 7, 99]))                        # integers: ids by sorted label
    assert G == 3 and ids.tolist() == [1, 1, 0, 2]
    ids, G = contiguous_group_ids(torch.tensor([[3, 3], [1, 3]]))
    assert G == 2 and ids.tolist() == [1, 1, 0, 1]
    ids, G = contiguous_group_ids(np.array(["u-1", "u-2", "u-1", 5, 5.0], dtype=object))
    assert G == 3 and ids.tolist() == [0, 1, 0, 2, 2]                               # Python equality: 5 == 5.0
    ids, G = contiguous_group_ids(["0042", 42, "x"])
    assert G == 3
    ids, G = contiguous_group_ids(["0042", "42", "7"], vectorized=True)             # numeric strings coincide there
    assert G == 2 and ids.tolist() == [1, 1, 0]                                     # integers again: by sorted label


def test_backward_rejects_operands_beyond_32_bit_offsets(lib):
    """The check runs before any GPU call: dummy non-null pointers are never dereferenced."""
    p = ctypes.c_void_p(256)
    rc = lib.vamd_lce_backward(p, p, p, 700000, 3584, 1024, 1.0, p, p, None, None, 0.0, None, p, p, 0, None, 0, p, 1 << 40, None)
    assert rc == -1 and b"4 GiB" in lib.vamd_last_error()
    # fp32 accumulation of the weight gradient needs its buffer; an unknown mode is refused
    rc = lib.vamd_lce_backward(p, p, p, 256, 128, 1024, 1.0, p, p, None, None, 0.0, None, p, None, 3, None, 0, p, 1 << 40, None)
    assert rc == -1 and b"d_weight_acc32" in lib.vamd_last_error()
    rc = lib.vamd_lce_backward(p, p, p, 256, 128, 1024, 1.0, p, p, None, None, 0.0, None, p, p, 7, None, 0, p, 1 << 40, None)
    assert rc == -1 and b"d_weight_mode" in lib.vamd_last_error()
    # a vocabulary that is not a multiple of 8 is served, but not together with a logits cache
    rc = lib.vamd_lce_forward(p, p, p, 256, 128, 1001, 1.0, p, p, p, p, p, None, p, 1 << 30, None)
    assert rc == -1 and b"multiple of 8" in lib.vamd_last_error()


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode != 0 and "one GPU" in res.stderr and res.stdout.strip() == ""


def test_static_forward_refuses_sizes_beyond_its_buffer_before_any_gpu_call(lib):
    # the pointers are never dereferenced: the size check precedes every HIP call
    rc = lib.vamd_lce_forward_static(1, 1, 1, 65536 + 1, 128, 256, 1.0, 1, 1, 1, 1, None, None)
    assert rc == -1 and b"at most 65536 tokens" in lib.vamd_last_error()


def test_as_torch_index_agrees_with_the_oracle_restatement():
    """The product's label handling is written differently from the oracle's line-by-line restatement of
    verl/utils/groupwise.py:91-160; both must give the same ids on every kind of label."""
    import uuid

    from oracle import advantages as A
    from verl_amd.utils.groupwise import as_torch_index
    rng = np.random.default_rng(0)
    uuids = [str(uuid.UUID(int=int(x))) for x in rng.integers(0, 2**62, 9)]
    cases = [
        torch.tensor([3, 1, 3, 2]), torch.tensor([3, 1, 3], dtype=torch.int32), torch.tensor([True, False, True]),
        torch.tensor([1.0, 2.0, 1.0]), torch.tensor([1.0, 2.0000001, 1.0]), torch.tensor([0.5, 1.5, 0.5]),
        torch.tensor([1.0, 2.0], dtype=torch.bfloat16), torch.tensor([[1, 2], [2, 1]]),
        np.array([3, 3, 7]), np.array([1.0, 2.0, 1.0]), np.array([1.5, 2.5, 1.5]), np.array([True, False]),
        np.array(["5", "6", "5"]), np.array(uuids * 2, dtype=object), ["a", "b", "a", "c", "0042", 42],
        ["5", "6", "5"], [3, 1, 3], (1.0, 2.0), np.array([[1, 2], [2, 1]]), [("a", 1), ("b", 2), ("a", 1)],
    ]
    for case in cases:
        want = A.as_torch_index(case)
        got = as_torch_index(case)
        assert got.dtype == torch.long and got.dim() == 1
        assert torch.equal(got, want.cpu()), f"{case!r}: {got.tolist()} vs {want.tolist()}"
