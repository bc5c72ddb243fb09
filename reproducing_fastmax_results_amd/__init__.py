"""Fastmax attention hot path for MI355X (gfx950): hand-written HIP kernels behind
a C ABI (``include/fastmax_hip.h``), a torch binding named ``fastmax_cuda`` and
the reference's operator fronts in ``attention_mechanisms.score_function``."""
__version__ = "0.1.0"
