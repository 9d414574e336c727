"""Gradient transformations that sit directly on the fused Adam operator."""

from torchopt_amd.transform.scale_by_adam import ScaleByAdamState, scale_by_accelerated_adam

__all__ = ['ScaleByAdamState', 'scale_by_accelerated_adam']
