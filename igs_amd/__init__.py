"""igs_amd -- MI355X-native 2-D Gaussian splatting (forward + backward) behind the
KohakuBlueleaf/IGS function / autograd.Function / module interface.

`from igs_amd import GaussianSplatting2D, gaussian_splatting_2d` mirrors
`from igs.gs2d import GaussianSplatting2D, gaussian_splatting_2d` of the reference
(src/igs/__init__.py:1, README.md:19).
"""
from .gs2d import (  # noqa: F401
    GaussianSplatting2D,
    GaussianSplatting2DChunkedKernel,
    GaussianSplatting2DKernel,
    TorchGaussianSplatting2DChunked,
    TorchGaussianSplatting2DKernel,
    gaussian_splatting_2d,
    naive_gaussian_2d,
)

from ._splat import exact, library_options  # noqa: F401,E402
from .fit import GaussianImageFit  # noqa: F401,E402
from .reg import koleo_diversity_loss  # noqa: F401,E402

__all__ = [
    "exact",
    "library_options",
    "GaussianImageFit",
    "koleo_diversity_loss",
    "GaussianSplatting2D",
    "gaussian_splatting_2d",
    "naive_gaussian_2d",
    "GaussianSplatting2DKernel",
    "TorchGaussianSplatting2DKernel",
    "TorchGaussianSplatting2DChunked",
    "GaussianSplatting2DChunkedKernel",
]
