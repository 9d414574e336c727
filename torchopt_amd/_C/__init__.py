"""Counterpart of the reference's native module ``torchopt._C``
(/root/reference/src/extension.cpp:20): one submodule, ``adam_op``."""

from torchopt_amd._C import adam_op

__all__ = ['adam_op']
