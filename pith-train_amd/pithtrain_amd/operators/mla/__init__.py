"""MLA / chunk attention operators. The reference picks a backend per NVIDIA architecture here
(pithtrain/operators/mla/__init__.py:3-11); this package has exactly one backend, the HIP kernels."""

from pithtrain_amd.operators.mla.hip import MLA, attention_func

__all__ = ["MLA", "attention_func"]
