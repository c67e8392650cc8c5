"""verl_amd: MI355X-native kernels for verl's per-token policy-math path.

The package mirrors the module paths of the reference for the functions it replaces:

    verl_amd.utils.kernel.linear_cross_entropy   <- verl.utils.kernel.linear_cross_entropy
    verl_amd.utils.torch_functional              <- verl.utils.torch_functional (masked_*)
    verl_amd.utils.groupwise                     <- verl.utils.groupwise
    verl_amd.trainer.ppo.core_algos              <- verl.trainer.ppo.core_algos (GAE, GRPO,
                                                    agg_loss, vanilla policy loss, value loss)

Every function runs hand-written HIP kernels from ``libverl_amd.so`` through a C ABI
(``include/verl_amd.h``).  There is no CPU or PyTorch fallback: without the built library or
without a GPU the calls raise.
"""

__version__ = "0.1.0"
