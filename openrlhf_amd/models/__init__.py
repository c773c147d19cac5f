"""The loss modules under the names ``openrlhf.models`` exports them (openrlhf/models/__init__.py);
the model classes of that package (Actor, reward / critic heads) are not part of this library."""
from .loss import (  # noqa: F401
    DPOLoss,
    GPTLMLoss,
    LogExpLoss,
    PairWiseLoss,
    PolicyLoss,
    SFTLoss,
    ValueLoss,
    aggregate_loss,
)

__all__ = ["DPOLoss", "GPTLMLoss", "LogExpLoss", "PairWiseLoss", "PolicyLoss", "SFTLoss", "ValueLoss", "aggregate_loss"]
