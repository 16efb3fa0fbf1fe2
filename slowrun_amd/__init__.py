"""MI355X-native fused fp8 LM-head + tanh-softcap + cross-entropy.

The compute lives in hand-written HIP kernels behind the C-ABI library
``libslowrun_ce.so`` (sources in ``slowrun_amd/csrc``); ``cuda_kernels`` mirrors
the module of the same name in the reference so a trainer can import
``FusedSoftcappedCrossEntropy`` and ``CE_KERNEL_VOCAB_SIZE`` from it unchanged.
"""
__version__ = "0.1.0"
