"""slayerpytorch_amd: SLAYER's per-neuron temporal kernels for AMD MI355X (gfx950).

``slayerCuda`` / ``slayerLoihiCuda`` are drop-in replacements of the reference's two extension
modules, bound to hand-written HIP kernels through the C ABI of ``libslayer_hip.so``;
``layer`` / ``loihi`` are the host-side layer engines that wrap them in autograd Functions;
``loss`` holds the spike-train losses built on the PSP kernel; ``synapse`` the per-timestep
convolution / pooling synapses; ``io`` the spike event files and their binning on the GPU;
``utils.capturedStep`` replays a whole training step from a HIP graph.
"""
from . import slayerCuda, slayerLoihiCuda            # noqa: F401
from .slayer import spikeLayer as layer               # noqa: F401
from .slayerLoihi import spikeLayer as loihi          # noqa: F401
from .slayerLoihi import quantize                     # noqa: F401
from .spikeLoss import spikeLoss as loss              # noqa: F401
from . import spikeFileIO as io                       # noqa: F401
from . import synapse                                 # noqa: F401
from . import utils                                   # noqa: F401

__all__ = ["slayerCuda", "slayerLoihiCuda", "layer", "loihi", "quantize", "loss", "io", "synapse", "utils"]
