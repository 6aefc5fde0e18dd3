"""Policy-gradient loss around the model (the caller side of the MXFP8 linear path in RL training)."""
from .loss import compute_policy_gradient_loss, compute_token_log_probs, token_log_probs

__all__ = ["compute_policy_gradient_loss", "compute_token_log_probs", "token_log_probs"]
