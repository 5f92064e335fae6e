"""FALKON kernel ridge regression with every K_nm / K_nm^T product routed through the F3M engine.

Same class names and call signatures as the reference's conjugate_gradient/ package
(custom_GaussianKernel, custom_Falkon, FalkonConjugateGradient_custom, ConjugateGradient), without
its dependency on the third-party ``falkon`` package: options and the preconditioner are provided
here (falkon is not pinned anywhere in the reference, so its defaults are chosen values).
"""
from .options import FalkonOptions, ConjugateGradientOptions
from .preconditioner import FalkonPreconditioner
from .custom_gaussian_kernel import custom_GaussianKernel
from .custom_conjugate_gradient_falkon import ConjugateGradient, FalkonConjugateGradient_custom
from .custom_falkon import custom_Falkon

__all__ = ["FalkonOptions", "ConjugateGradientOptions", "FalkonPreconditioner", "custom_GaussianKernel",
           "ConjugateGradient", "FalkonConjugateGradient_custom", "custom_Falkon"]
