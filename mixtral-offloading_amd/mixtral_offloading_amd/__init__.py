"""MI355X-native HQQ quantized-linear hot path with the module surface of
dvmazur/mixtral-offloading (``HQQLinearTritonSavable``, ``MixtralExpertWrapper``,
``ExpertCache``, ``build_model``).  All arithmetic runs in the HIP library
``libhqq_mi355x.so`` reached through its C ABI; there is no CPU fallback."""

from . import _lib  # noqa: F401  (fails loudly when the HIP library is missing)
