"""MI355X (gfx950) backend of the fused linear-logprob path.

Python mirror of the reference operator interface (kernel registry + op classes) over the C-ABI
library ``librlk_hip.so``.  Everything numerical runs in hand-written HIP kernels; this package
only validates arguments, allocates tensors and forwards raw pointers.
"""

__version__ = "0.1.0"
