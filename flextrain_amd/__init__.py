"""flextrain_amd: MI355X (gfx950) implementation of FlexTrain's per-layer
training compute path behind FlexTrain's own ``flextrain_*`` op signatures.

Importing this package touches neither the GPU nor the native library; the
library is loaded on the first op call (``flextrain_amd._lib.lib()``), so test
collection and CPU-only tooling work without a device.
"""

__version__ = "0.1"
