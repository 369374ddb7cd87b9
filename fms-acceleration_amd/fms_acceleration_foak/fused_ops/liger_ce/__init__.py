from .fused_linear_cross_entropy_loss import (  # noqa: F401
    LigerFusedLinearCrossEntropyFunction,
    LigerFusedLinearCrossEntropyLoss,
    lce_forward,
)
