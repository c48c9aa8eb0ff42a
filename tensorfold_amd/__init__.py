"""MI355X-native kernels behind TensorFold's quantized routed-expert matmul call surface.

Modules mirror the reference's: ``qmm`` (cuda/kernels/qmm.py), ``experts`` (cuda/experts.py), ``moe`` (cuda/moe.py),
``exl3.linear`` / ``exl3.format`` (cuda/exl3/), ``build`` (cuda/build.py).  Every op calls hand-written HIP kernels
for gfx950 through the C ABI of ``libtfmi.so`` (``include/tfmi.h``); there is no CPU or PyTorch fallback.
"""

__version__ = "0.1.0"
