"""pithtrain_amd — MI355X (gfx950) implementation of PithTrain's context-parallel ring-attention
hot path: hand-written HIP kernels behind a flat C ABI (libpith_hip.so), called from PyTorch-ROCm
host code that keeps the reference operators' Python signatures.

Layout (mirrors pithtrain/operators/ of the reference):
    operators/mla/hip.py                 _mla_fwd, _mla_bwd_preprocess, _mla_bwd_dk_dv, _mla_bwd_dq, MLA
    operators/ring_attention/mla.py      _online_softmax_combine_log2, RingMLAAttentionFunc, ring_mla_attention_func
    operators/ring_attention/standard.py _online_softmax_combine, RingAttentionFunc, ring_attention_func
    operators/ring_attention/local.py    collective-free one-GPU ring drivers (contiguous and zigzag schedules)
"""

__version__ = "0.1.0"
