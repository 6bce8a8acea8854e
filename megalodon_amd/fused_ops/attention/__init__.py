from .softmax import attention_softmax
from .swift import (swift_efficient_attention, swift_efficient_attention_bwd,
                    swift_efficient_attention_fwd)

__all__ = ["attention_softmax", "swift_efficient_attention", "swift_efficient_attention_fwd",
           "swift_efficient_attention_bwd"]
