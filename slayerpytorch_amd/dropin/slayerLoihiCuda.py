"""Top-level ``slayerLoihiCuda`` module for unmodified reference code
(``import slayerLoihiCuda``): put this directory on ``sys.path`` instead of installing the
CUDA extension."""
from slayerpytorch_amd.slayerLoihiCuda import getSpikes   # noqa: F401
