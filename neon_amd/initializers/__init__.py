"""Parameter initialisers: host-side draws written into device tensors."""
from neon_amd.initializers.initializer import (Array, Constant, Gaussian, GlorotUniform, IdentityInit,  # noqa: F401
                                               Initializer, Kaiming, Orthonormal, Uniform, Xavier)
