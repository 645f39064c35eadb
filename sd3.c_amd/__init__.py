"""MI355X-native SD3.5-medium MMDiT-X denoiser forward behind the module API of MichelHUANGGit/SD3.c.

Importing the package does not touch the GPU. `sd3_c_amd.modules` (the mirror of the reference's
`custom_modules` extension) loads the HIP library on first use and raises if it is missing.
"""
from .config import DiTConfig, sd35_medium, reference_dit_test  # noqa: F401
from . import params  # noqa: F401
