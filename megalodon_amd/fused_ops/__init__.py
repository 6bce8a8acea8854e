"""Fused ops with the reference's names (megalodon/modules/fused_ops/__init__.py:1-14)."""
from .attention import (attention_softmax, swift_efficient_attention, swift_efficient_attention_bwd,
                        swift_efficient_attention_fwd)
from .block_glue import layer_norm_plus_one, qk_norm_rotary, silu_mul, transpose_last2
from .cema_kernel import cema_kernel
from .cema_scan import cema_scan, cema_scan_applicable, cema_scan_state
from .ema_hidden import ema_hidden
from .ema_parameters import ema_parameters
from .fftconv import fftconv, fftconv_residual, fused_fftconv_bwd, fused_fftconv_fwd
from .sequence_norm import sequence_norm
from .memory_efficient_dropout import (memory_efficient_dropout, memory_efficient_dropout_bwd,
                                       memory_efficient_dropout_fwd)

__all__ = ["attention_softmax", "cema_kernel", "cema_scan", "cema_scan_applicable", "cema_scan_state", "ema_hidden", "ema_parameters", "fftconv", "fftconv_residual", "sequence_norm", "fused_fftconv_fwd", "fused_fftconv_bwd",
           "memory_efficient_dropout", "memory_efficient_dropout_fwd", "memory_efficient_dropout_bwd",
           "swift_efficient_attention", "swift_efficient_attention_fwd",
           "swift_efficient_attention_bwd", "silu_mul", "transpose_last2", "layer_norm_plus_one", "qk_norm_rotary"]
