"""Plain-PyTorch statement of the fused Adam operator (see `adam_op`): a readable cross-check, never
a fallback -- nothing in `torchopt_amd` imports it on its own."""
