from .cross_entropy import (LigerCrossEntropyFunction, LigerForCausalLMLoss, cross_entropy_backward,
                            cross_entropy_forward, liger_fixed_cross_entropy)
