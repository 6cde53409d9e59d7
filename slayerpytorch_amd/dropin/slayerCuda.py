"""Top-level ``slayerCuda`` module for unmodified reference code (``import slayerCuda``):
put this directory on ``sys.path`` instead of installing the CUDA extension."""
from slayerpytorch_amd.slayerCuda import *            # noqa: F401,F403
from slayerpytorch_amd.slayerCuda import getSpikes, conv, corr, shift   # noqa: F401
