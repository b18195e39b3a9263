"""MI355X-native implementation of the MoEspresso attention hot path.

Python operator modules under ``moespresso_amd.runtime`` mirror the reference's
``moespresso.runtime.deepseek_v4`` / ``moespresso.runtime.qwen`` callables on
``torch.Tensor`` inputs and call hand-written gfx950 kernels through the C-ABI
of ``libmoespresso_amd.so`` (declared in ``include/moespresso_amd.h``).
"""

__version__ = "0.1.0"
