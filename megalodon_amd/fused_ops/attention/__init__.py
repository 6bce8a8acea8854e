from .swift import (swift_efficient_attention, swift_efficient_attention_bwd,
                    swift_efficient_attention_fwd)

__all__ = ["swift_efficient_attention", "swift_efficient_attention_fwd", "swift_efficient_attention_bwd"]
