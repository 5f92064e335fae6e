"""Options of the FALKON drivers.  The reference takes them from the third-party ``falkon`` package
(``falkon.options``; used at conjugate_gradient/custom_conjugate_gradient_falkon.py:56,74,84), whose
version is pinned nowhere in the reference; the defaults below are this package's chosen values."""
import dataclasses

import torch


@dataclasses.dataclass
class ConjugateGradientOptions:
    cg_epsilon_32: float = 1e-7          # added to denominators in fp32
    cg_epsilon_64: float = 1e-15
    cg_tolerance: float = 1e-7           # stop when sqrt(max residual norm^2) falls below
    cg_full_gradient_every: int = 10     # recompute R = B - A X every this many iterations

    def cg_epsilon(self, dtype):
        return self.cg_epsilon_32 if dtype == torch.float32 else self.cg_epsilon_64


@dataclasses.dataclass
class FalkonOptions(ConjugateGradientOptions):
    pc_epsilon_32: float = 1e-5          # jitter (times M) added to K_MM before its Cholesky, fp32 data
    pc_epsilon_64: float = 1e-13
    pc_dtype: torch.dtype = torch.float64   # precision of the preconditioner factors
    # keep T^-1 and A^-1 as dense matrices (two more M x M matrices) so that every triangular solve of
    # the conjugate-gradient loop becomes one matrix-vector product; off: back-substitution each time
    pc_explicit_inverse: bool = True
    # Preconditioner factorised, multiplied and solved tile by tile in fp32 storage (diagonal tiles in fp64), so
    # that no library call sees more than pc_block_size^2 entries: None = whenever a matrix in pc_dtype would
    # exceed the limit for whole-matrix calls (the benchmark's M = 1e5), True = always, False = never
    pc_blocked: object = None
    pc_block_size: int = 8192
    use_cpu: bool = False                # kept for signature compatibility; the engine is GPU only
    debug: bool = False

    def get_conjgrad_options(self):
        return ConjugateGradientOptions(self.cg_epsilon_32, self.cg_epsilon_64, self.cg_tolerance,
                                        self.cg_full_gradient_every)

    def pc_epsilon(self, dtype):
        return self.pc_epsilon_32 if dtype == torch.float32 else self.pc_epsilon_64
